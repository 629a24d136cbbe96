// Conv2d forward and weight gradient for stride 1, dilation 1: the input patch of an output tile is staged
// in LDS once and every kernel tap reads it from there.
//
// l-ten writes an im2col buffer per image and multiplies it with the weight matrix (l-ten/conv2d.cpp:164-171
// forward, l-ten/backprop.cpp:1949-1953 weight gradient); the buffer repeats every input element kh*kw times.
// Here a workgroup loads the rows of x that its output tile touches (tile + halo) into LDS, and the MFMA
// operand of tap (i, j) is the same LDS patch read at an offset of i rows and j columns, so x crosses the
// memory system once per tile instead of kh*kw times and no index arithmetic runs per element.
//
// The reduction index of a product is free to be reordered as long as both operands agree.  Both kernels
// order it so that the two reduction positions one v_mfma_f32_32x32x2f32 consumes (lanes 0-31 and 32-63)
// differ by a fixed LDS stride: then every operand address is one per-lane base plus an immediate.
#include "conv_common.h"
#include "gemm_f32_core.h"

#include <algorithm>
#include <type_traits>

namespace lten_hip {

// ---------------------------------------------------------------------------------------------------------
// Forward.  Workgroup tile: BM = 64 (or 32) output channels x (TH = 4 rows x TW = 128 columns) of one image;
// wavefront `wave` owns row `wave` (BM / 32 x 4 MFMA tiles of 32 x 32).  The input channels are walked in chunks of CB = 4:
// per chunk the patch [4][TH + KH - 1][PWS] and the weights of those channels are stored to LDS, the next
// chunk's values are fetched to registers, and (CB / 2) * KH * KW MFMA steps run; step (cp, i, j) multiplies
// tap (i, j) of channels 2cp (lanes 0-31) and 2cp + 1 (lanes 32-63).
//
// LDS patch row: index q holds input column w0 - 4 + q (interior 16-byte aligned, left halo in 4 - pw .. 3).
// LDS weights: [step][channel parity][WROW = BM + 1] (the odd row length spreads the scattered stores over banks).
template <int KH, int KW, int BM_>
struct PatchFwd {
	static constexpr int CB = 4, TH = 4, TW = 128, NT = TW / 32, BM = BM_, MT = BM / 32, T = 256;
	static constexpr int PR = TH + KH - 1;
	static constexpr int PWS = (4 + TW + KW - 1 + 3) / 4 * 4;
	static constexpr int F4_ROW = PWS / 4;
	static constexpr int PATCH = CB * PR * PWS;
	static constexpr int PATCH_F4 = CB * PR * F4_ROW;
	static constexpr int P_PER_T = (PATCH_F4 + T - 1) / T;
	static constexpr int TAPS = KH * KW;
	static constexpr int KSTEPS = (CB / 2) * TAPS;
	static constexpr int WROW = BM + 1;
	static constexpr int WTS = KSTEPS * 2 * WROW;
	static constexpr int WCOUNT = BM * CB * TAPS;
	static constexpr int W_PER_T = (WCOUNT + T - 1) / T;
};

template <int KH, int KW, int BM, bool VEC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(BM == 64 ? 2 : 3, BM == 64 ? 2 : 3))) void conv2d_patch_forward_kernel(
    ConvGeo g, const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ y)
{
	typedef PatchFwd<KH, KW, BM> P;
	__shared__ __attribute__((aligned(16))) float s_patch[P::PATCH];
	__shared__ float s_w[P::WTS];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lrow = lane & 31, half = lane >> 5;
	const int tiles_w = (g.Wo + P::TW - 1) / P::TW;
	const int w0 = (int)(blockIdx.x % tiles_w) * P::TW, h0 = (int)(blockIdx.x / tiles_w) * P::TH;
	const int co0 = blockIdx.y * P::BM, n = blockIdx.z;
	const int Kc = g.Cin * P::TAPS;
	const float* xn = x + (int64_t)n * g.Cin * g.H * g.W;

	float4 rp[P::P_PER_T];
	float rw[P::W_PER_T];
	auto load_chunk = [&](int c0) {
#pragma unroll
		for (int q = 0; q < P::P_PER_T; q++) {
			const int idx = tid + q * P::T;
			const int f = idx % P::F4_ROW, rowid = idx / P::F4_ROW;
			const int pr = rowid % P::PR, c = rowid / P::PR;
			const int gy = h0 + pr - g.ph;
			float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			if (idx < P::PATCH_F4 && c0 + c < g.Cin && gy >= 0 && gy < g.H)
				v = load_row4<VEC>(xn + ((int64_t)(c0 + c) * g.H + gy) * g.W, w0 - 4 + 4 * f, g.W);
			rp[q] = v;
		}
#pragma unroll
		for (int q = 0; q < P::W_PER_T; q++) {
			const int idx = tid + q * P::T;
			const int co = idx / (P::CB * P::TAPS), kk = idx % (P::CB * P::TAPS);
			const int k = c0 * P::TAPS + kk;
			rw[q] = (idx < P::WCOUNT && co0 + co < g.Cout && k < Kc) ? w[(int64_t)(co0 + co) * Kc + k] : 0.0f;
		}
	};
	auto store_chunk = [&]() {
#pragma unroll
		for (int q = 0; q < P::P_PER_T; q++) {
			const int idx = tid + q * P::T;
			if (idx < P::PATCH_F4) *reinterpret_cast<float4*>(s_patch + idx * 4) = rp[q];
		}
#pragma unroll
		for (int q = 0; q < P::W_PER_T; q++) {
			const int idx = tid + q * P::T;
			const int co = idx / (P::CB * P::TAPS), kk = idx % (P::CB * P::TAPS);
			const int c = kk / P::TAPS, tap = kk % P::TAPS;
			if (idx < P::WCOUNT) s_w[(((c >> 1) * P::TAPS + tap) * 2 + (c & 1)) * P::WROW + co] = rw[q];
		}
	};

	v16f acc[P::MT][P::NT];
#pragma unroll
	for (int m = 0; m < P::MT; m++)
#pragma unroll
		for (int t = 0; t < P::NT; t++)
#pragma unroll
			for (int r = 0; r < 16; r++) acc[m][t][r] = 0.0f;

	const float* pa = s_w + half * P::WROW + lrow;
	const float* pb = s_patch + (half * P::PR + wave) * P::PWS + lrow + 4 - g.pw;

	load_chunk(0);
	for (int c0 = 0; c0 < g.Cin; c0 += P::CB) {
		store_chunk();
		__syncthreads();
		if (c0 + P::CB < g.Cin) load_chunk(c0 + P::CB);
		// operands of step s + 1 are read while the MFMAs of step s issue, one LDS read behind each MFMA
		constexpr int NR = P::MT + P::NT, NM = P::MT * P::NT;  // LDS reads and MFMAs per step
		float fa[2][P::MT], fb[2][P::NT];
		auto read_operand = [&](int s, int e) {
			const int cp = s / P::TAPS, tap = s % P::TAPS, i = tap / KW, j = tap % KW;
			if (e < P::MT) fa[s & 1][e] = pa[s * 2 * P::WROW + e * 32];
			else fb[s & 1][e - P::MT] = pb[(2 * cp * P::PR + i) * P::PWS + j + (e - P::MT) * 32];
		};
#pragma unroll
		for (int e = 0; e < NR; e++) read_operand(0, e);
#pragma unroll
		for (int s = 0; s < P::KSTEPS; s++) {
#pragma unroll
			for (int e = 0; e < NM; e++) {
				acc[e / P::NT][e % P::NT] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s & 1][e / P::NT], fb[s & 1][e % P::NT], acc[e / P::NT][e % P::NT], 0, 0, 0);
				if (s + 1 < P::KSTEPS) {
					if (e < NR) read_operand(s + 1, e);
					if (e == NM - 1)
						for (int x = NM; x < NR; x++) read_operand(s + 1, x);
				}
				__builtin_amdgcn_sched_barrier(0);
			}
		}
		__syncthreads();
	}

	// Epilogue.  All bias values are loaded before the first store, so that no store waits behind a load; an
	// address is a part the wavefront shares (row ho of channel co0 + 32m + 8(r/4) + r%4) plus a lane offset.
	const int ho = h0 + __builtin_amdgcn_readfirstlane(wave);
	if (ho >= g.Ho) return;
	float bv[P::MT][16];
#pragma unroll
	for (int m = 0; m < P::MT; m++)
#pragma unroll
		for (int r = 0; r < 16; r++) {
			const int co = co0 + m * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
			bv[m][r] = (bias && co < g.Cout) ? bias[co] : 0.0f;
		}
	const int64_t plane = (int64_t)g.Ho * g.Wo;
	float* yw = y + (((int64_t)n * g.Cout + co0) * g.Ho + ho) * g.Wo + w0;
	const unsigned y_lane = (unsigned)(half * 4 * plane) + lrow;
	if (co0 + P::BM <= g.Cout && w0 + P::TW <= g.Wo) {
#pragma unroll
		for (int m = 0; m < P::MT; m++)
#pragma unroll
			for (int r = 0; r < 16; r++) {
				float* yr = yw + (m * 32 + (r >> 2) * 8 + (r & 3)) * plane;
#pragma unroll
				for (int t = 0; t < P::NT; t++) yr[y_lane + t * 32] = acc[m][t][r] + bv[m][r];
			}
		return;
	}
#pragma unroll
	for (int m = 0; m < P::MT; m++)
#pragma unroll
		for (int r = 0; r < 16; r++) {
			if (co0 + m * 32 + (r >> 2) * 8 + half * 4 + (r & 3) >= g.Cout) continue;
			float* yr = yw + (m * 32 + (r >> 2) * 8 + (r & 3)) * plane;
#pragma unroll
			for (int t = 0; t < P::NT; t++)
				if (w0 + t * 32 + lrow < g.Wo) yr[y_lane + t * 32] = acc[m][t][r] + bv[m][r];
		}
}

// ---------------------------------------------------------------------------------------------------------
// Weight gradient.  dw[co][ci][i][j] = sum over (n, ho, wo) of dy[n][co][ho][wo] * x[n][ci][ho+i-ph][wo+j-pw].
// As a product: rows = 64 output channels, columns = (tap, 32 input channels), reduction over output pixels.
// A workgroup owns a co block, a ci block and a contiguous range of chunks (a chunk = TW = 64 pixels of one
// output row); per chunk it stages dy[64][64] and the patch [32 ci][KH rows][PWS] in LDS.  Wavefront
// (mt, ph) multiplies MFMA row tile mt against all KH*KW tap tiles over pixel half ph of the chunk; one
// MFMA step takes pixels 2s (lanes 0-31) and 2s + 1 (lanes 32-63).  At the end the two pixel halves are added
// through LDS and the workgroup writes one partial [Cout][Cin*KH*KW] block; a second kernel adds the parts.
// V2: the chunk for narrow images, two rows of 32 pixels (pixel p of the chunk: row p / 32, column p % 32): the patch has
// one row more and 32 columns less.  A 28 x 28 image fills 7/8 of such chunks, against 7/16 of the 64-pixel row segments.
template <int KH, int KW, bool V2 = false>
struct PatchWgrad {
	static constexpr int BM = 64, CIB = 32, TW = 64, T = 256, TAPS = KH * KW;
	static constexpr int CW = V2 ? 32 : 64, CR = V2 ? 2 : 1;  // columns and rows of a chunk
	static constexpr int PROWS = KH + CR - 1;                // patch rows
	static constexpr int PWS = (4 + CW + KW - 1 + 3) / 4 * 4;
	static constexpr int F4_ROW = PWS / 4;
	static constexpr int CS = (PROWS * PWS) | 1;  // odd channel stride: 32 channels hit 32 banks
	static constexpr int DYS = TW + 1;
	static constexpr int DY_FLOATS = BM * DYS, PATCH_FLOATS = CIB * CS;
	static constexpr int LDS_FLOATS = DY_FLOATS + PATCH_FLOATS;
	static constexpr int DY_F4 = BM * TW / 4, DY_PER_T = DY_F4 / T;
	static constexpr int PATCH_F4 = CIB * PROWS * F4_ROW, P_PER_T = (PATCH_F4 + T - 1) / T;
	static constexpr int TAPS_PER_ROUND = LDS_FLOATS / (2 * 64 * 16);  // taps whose accumulators fit the final exchange
	static_assert(DY_F4 % T == 0 && TAPS_PER_ROUND >= 1, "tile shape");
};

// PIPE: one workgroup per CU with two LDS buffers.  The tiles of chunk c + 1 are stored to the other buffer during
// the last third of chunk c's MFMAs, one 4-byte store behind each MFMA, so that the matrix pipe does not wait while
// a workgroup refills its tiles, and a chunk costs one barrier.  Without PIPE: two workgroups per CU, one buffer,
// store - barrier - multiply - barrier (each workgroup's refill is meant to hide behind the other's MFMAs, which
// works only when the two are out of step).
template <int KH, int KW, bool VEC, bool PIPE, bool V2 = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(PIPE ? 1 : 2, PIPE ? 1 : 2))) void conv2d_patch_wgrad_kernel(
    ConvGeo g, const float* __restrict__ x, const float* __restrict__ dy, float* __restrict__ partial, int chunks_per_part)
{
	typedef PatchWgrad<KH, KW, V2> P;
	static_assert(!V2 || VEC, "the two-row chunk is loaded 16 bytes at a time");
	__shared__ float lds[(PIPE ? 2 : 1) * P::LDS_FLOATS];
	float* s_dy = lds;
	float* s_patch = lds + P::DY_FLOATS;

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lrow = lane & 31, half = lane >> 5;
	const int mt = wave & 1, phalf = wave >> 1;
	const int co0 = blockIdx.y * P::BM, ci0 = blockIdx.z * P::CIB;
	const int tiles_w = (g.Wo + P::CW - 1) / P::CW, rows_c = (g.Ho + P::CR - 1) / P::CR;
	const int total = g.N * rows_c * tiles_w;
	const int begin = blockIdx.x * chunks_per_part, end = min(total, begin + chunks_per_part);

	float4 rdy[P::DY_PER_T], rp[P::P_PER_T];
	// What does not change from chunk to chunk is worked out once per lane: the offset of each of its float4s from
	// the chunk's origin, and the row / column shifts that decide whether the float4 lies inside the image (with
	// VEC, rows are whole float4s: inside or outside together).  Chunk coordinates advance without divisions.
	int n_c = begin / (tiles_w * rows_c), ho_c = ((begin / tiles_w) % rows_c) * P::CR, w0_c = (begin % tiles_w) * P::CW;
	const int64_t plane_o = (int64_t)g.Ho * g.Wo;
	// this thread's float4 of a dy row of the chunk: pixels 4 (tid % 16) ..: row dy_r of the chunk, columns dy_c ..
	const int dy_r = (tid % (P::TW / 4)) / (P::CW / 4), dy_c = 4 * ((tid % (P::TW / 4)) % (P::CW / 4));
	const int dy_rel = (int)((tid / (P::TW / 4)) * plane_o) + dy_r * g.Wo + dy_c;  // + q * 16 rows of dy
	int x_rel[P::P_PER_T], x_gy[P::P_PER_T], x_gx[P::P_PER_T];
#pragma unroll
	for (int q = 0; q < P::P_PER_T; q++) {
		const int idx = tid + q * P::T;
		const int f = idx % P::F4_ROW, rowid = idx / P::F4_ROW;
		const int r = rowid % P::PROWS, ci = rowid / P::PROWS;
		const bool exists = idx < P::PATCH_F4 && ci0 + ci < g.Cin;
		x_gx[q] = 4 * f - 4;
		x_gy[q] = exists ? r - g.ph : -(1 << 30);
		x_rel[q] = exists ? (ci * g.H + r - g.ph) * g.W + x_gx[q] : 0;
	}
	auto load_chunk = [&]() {  // the chunk at (n_c, ho_c, w0_c)
		if (VEC) {
			const float* dyc = dy + (((int64_t)n_c * g.Cout + co0) * g.Ho + ho_c) * g.Wo + w0_c;
			const float* xc = x + (((int64_t)n_c * g.Cin + ci0) * g.H + ho_c) * g.W + w0_c;
			const bool dy_col = w0_c + dy_c < g.Wo && ho_c + dy_r < g.Ho;
#pragma unroll
			for (int q = 0; q < P::DY_PER_T; q++) {
				rdy[q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
				if (dy_col && co0 + tid / (P::TW / 4) + q * (P::T / (P::TW / 4)) < g.Cout)
					rdy[q] = *reinterpret_cast<const float4*>(dyc + dy_rel + q * (P::T / (P::TW / 4)) * plane_o);
			}
#pragma unroll
			for (int q = 0; q < P::P_PER_T; q++) {
				rp[q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
				if ((unsigned)(ho_c + x_gy[q]) < (unsigned)g.H && (unsigned)(w0_c + x_gx[q]) < (unsigned)g.W)
					rp[q] = *reinterpret_cast<const float4*>(xc + x_rel[q]);
			}
			return;
		}
		const int ho = ho_c, n = n_c, w0 = w0_c;
#pragma unroll
		for (int q = 0; q < P::DY_PER_T; q++) {
			const int idx = tid + q * P::T;
			const int p4 = idx % (P::TW / 4), co = idx / (P::TW / 4);
			float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			if (co0 + co < g.Cout) v = load_row4<VEC>(dy + (((int64_t)n * g.Cout + co0 + co) * g.Ho + ho) * g.Wo, w0 + 4 * p4, g.Wo);
			rdy[q] = v;
		}
#pragma unroll
		for (int q = 0; q < P::P_PER_T; q++) {
			const int idx = tid + q * P::T;
			const int f = idx % P::F4_ROW, rowid = idx / P::F4_ROW;
			const int r = rowid % KH, ci = rowid / KH;
			const int gy = ho + r - g.ph;
			float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			if (idx < P::PATCH_F4 && ci0 + ci < g.Cin && gy >= 0 && gy < g.H)
				v = load_row4<VEC>(x + (((int64_t)n * g.Cin + ci0 + ci) * g.H + gy) * g.W, w0 - 4 + 4 * f, g.W);
			rp[q] = v;
		}
	};
	auto next_chunk = [&]() {
		w0_c += P::CW;
		if (w0_c >= g.Wo) {
			w0_c = 0;
			ho_c += P::CR;
			if (ho_c >= g.Ho) { ho_c = 0; n_c++; }
		}
	};
	auto store_chunk = [&]() {
#pragma unroll
		for (int q = 0; q < P::DY_PER_T; q++) {
			const int idx = tid + q * P::T;
			float* d = s_dy + (idx / (P::TW / 4)) * P::DYS + 4 * (idx % (P::TW / 4));
			d[0] = rdy[q].x; d[1] = rdy[q].y; d[2] = rdy[q].z; d[3] = rdy[q].w;
		}
#pragma unroll
		for (int q = 0; q < P::P_PER_T; q++) {
			const int idx = tid + q * P::T;
			const int f = idx % P::F4_ROW, rowid = idx / P::F4_ROW;
			float* d = s_patch + (rowid / P::PROWS) * P::CS + (rowid % P::PROWS) * P::PWS + 4 * f;
			if (idx < P::PATCH_F4) { d[0] = rp[q].x; d[1] = rp[q].y; d[2] = rp[q].z; d[3] = rp[q].w; }
		}
	};

	v16f acc[P::TAPS];
#pragma unroll
	for (int t = 0; t < P::TAPS; t++)
#pragma unroll
		for (int r = 0; r < 16; r++) acc[t][r] = 0.0f;

	const float* pa = s_dy + (mt * 32 + lrow) * P::DYS + phalf * (P::TW / 2) + half;
	// pixel half phalf of the chunk: the second 32 columns of the row, or (V2) the second row
	const float* pb = s_patch + lrow * P::CS + (V2 ? phalf * P::PWS : phalf * (P::TW / 2)) + half + 4 - g.pw;

	if (PIPE) {
		// piece k of the 16 + 4 * P_PER_T four-byte stores that put this thread's share of a chunk into a buffer
		constexpr int PIECES = 4 * (P::DY_PER_T + P::P_PER_T), STEPS = P::TW / 4, SLOTS = STEPS * P::TAPS;
		static_assert(PIECES <= SLOTS, "one store behind each MFMA at most");
		int off_d[P::DY_PER_T], off_p[P::P_PER_T];
#pragma unroll
		for (int q = 0; q < P::DY_PER_T; q++) {
			const int idx = tid + q * P::T;
			off_d[q] = (idx / (P::TW / 4)) * P::DYS + 4 * (idx % (P::TW / 4));
		}
#pragma unroll
		for (int q = 0; q < P::P_PER_T; q++) {
			const int idx = tid + q * P::T;
			const int f = idx % P::F4_ROW, rowid = idx / P::F4_ROW;
			off_p[q] = idx < P::PATCH_F4 ? P::DY_FLOATS + (rowid / P::PROWS) * P::CS + (rowid % P::PROWS) * P::PWS + 4 * f : -1;
		}
		auto store_piece = [&](float* buf, int k) {
			if (k < 4 * P::DY_PER_T) {
				const float4 v = rdy[k / 4];
				buf[off_d[k / 4] + (k % 4)] = (k % 4) == 0 ? v.x : (k % 4) == 1 ? v.y : (k % 4) == 2 ? v.z : v.w;
			} else {
				const int kk = k - 4 * P::DY_PER_T;
				const float4 v = rp[kk / 4];
				if (off_p[kk / 4] >= 0) buf[off_p[kk / 4] + (kk % 4)] = (kk % 4) == 0 ? v.x : (kk % 4) == 1 ? v.y : (kk % 4) == 2 ? v.z : v.w;
			}
		};
		if (begin < end) {
			load_chunk();
#pragma unroll
			for (int k = 0; k < PIECES; k++) store_piece(lds, k);
			__syncthreads();
			next_chunk();
			if (begin + 1 < end) load_chunk();
		}
		// MORE: a chunk follows, whose tiles are stored to the other buffer on the way
		auto run_chunk = [&](int chunk, auto more_tag) {
			constexpr bool MORE = decltype(more_tag)::value;
			const int cur = (chunk - begin) & 1;
			const float* pac = pa + cur * P::LDS_FLOATS;
			const float* pbc = pb + cur * P::LDS_FLOATS;
			float* other = lds + (cur ^ 1) * P::LDS_FLOATS;
			float fa[2], fb[2][P::TAPS];
			auto read_operand = [&](int s, int t) { fb[s & 1][t] = pbc[(t / KW) * P::PWS + (t % KW) + 2 * s]; };
			fa[0] = pac[0];
#pragma unroll
			for (int t = 0; t < P::TAPS; t++) read_operand(0, t);
#pragma unroll
			for (int s = 0; s < STEPS; s++) {
#pragma unroll
				for (int t = 0; t < P::TAPS; t++) {
					acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s & 1], fb[s & 1][t], acc[t], 0, 0, 0);
					if (s + 1 < STEPS) {
						if (t == 0) fa[(s + 1) & 1] = pac[2 * (s + 1)];
						read_operand(s + 1, t);
					}
					const int k = s * P::TAPS + t - (SLOTS - PIECES);
					if (MORE && k >= 0) store_piece(other, k);
					__builtin_amdgcn_sched_barrier(0);
				}
			}
			// the registers are free again: fetch the chunk after next, then let everybody finish with both buffers
			next_chunk();
			if (chunk + 2 < end) load_chunk();
			__syncthreads();
		};
		for (int chunk = begin; chunk + 1 < end; chunk++) run_chunk(chunk, std::true_type{});
		if (begin < end) run_chunk(end - 1, std::false_type{});
	} else {
	if (begin < end) load_chunk();
	for (int chunk = begin; chunk < end; chunk++) {
		store_chunk();
		__syncthreads();
		next_chunk();
		if (chunk + 1 < end) load_chunk();
		// operands of step s + 1 are read while the MFMAs of step s issue
		float fa[2], fb[2][P::TAPS];
		auto read_operand = [&](int s, int t) { fb[s & 1][t] = pb[(t / KW) * P::PWS + (t % KW) + 2 * s]; };
		fa[0] = pa[0];
#pragma unroll
		for (int t = 0; t < P::TAPS; t++) read_operand(0, t);
#pragma unroll
		for (int s = 0; s < P::TW / 4; s++) {
#pragma unroll
			for (int t = 0; t < P::TAPS; t++) {
				acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s & 1], fb[s & 1][t], acc[t], 0, 0, 0);
				if (s + 1 < P::TW / 4) {
					if (t == 0) fa[(s + 1) & 1] = pa[2 * (s + 1)];
					read_operand(s + 1, t);
				}
				__builtin_amdgcn_sched_barrier(0);
			}
		}
		__syncthreads();
	}
	}

	// pixel half 1 hands its sums to pixel half 0 of the same row tile, TAPS_PER_ROUND taps at a time
#pragma unroll
	for (int t0 = 0; t0 < P::TAPS; t0 += P::TAPS_PER_ROUND) {
		if (phalf == 1) {
#pragma unroll
			for (int t = t0; t < t0 + P::TAPS_PER_ROUND && t < P::TAPS; t++)
#pragma unroll
				for (int r = 0; r < 16; r++) lds[((mt * P::TAPS_PER_ROUND + (t - t0)) * 16 + r) * 64 + lane] = acc[t][r];
		}
		__syncthreads();
		if (phalf == 0) {
#pragma unroll
			for (int t = t0; t < t0 + P::TAPS_PER_ROUND && t < P::TAPS; t++)
#pragma unroll
				for (int r = 0; r < 16; r++) acc[t][r] += lds[((mt * P::TAPS_PER_ROUND + (t - t0)) * 16 + r) * 64 + lane];
		}
		__syncthreads();
	}
	if (phalf != 0) return;

	const int Kc = g.Cin * P::TAPS;
	float* out = partial + (int64_t)blockIdx.x * g.Cout * Kc;
	const int ci = ci0 + lrow;
	if (ci >= g.Cin) return;
#pragma unroll
	for (int r = 0; r < 16; r++) {
		const int co = co0 + mt * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
		if (co >= g.Cout) continue;
#pragma unroll
		for (int t = 0; t < P::TAPS; t++) out[(int64_t)co * Kc + ci * P::TAPS + t] = acc[t][r];
	}
}

// out[i] = sum over parts of partial[p][i].  A workgroup takes OUTS outputs; its 1024 / OUTS groups of lanes each
// add every GROUPS-th part (eight loads in flight, added in part order), then the group sums are added in
// group order.  Few outputs (a first layer's weights) get the narrow shape, so that more than a handful of
// workgroups share the reading.
template <int OUTS>
__global__ __launch_bounds__(1024) void conv_reduce_partials_kernel(const float* __restrict__ partial, int parts, int64_t count, float* __restrict__ out)
{
	constexpr int GROUPS = 1024 / OUTS;
	__shared__ float s[GROUPS][OUTS];
	const int o = threadIdx.x % OUTS, grp = threadIdx.x / OUTS;
	const int64_t idx = (int64_t)blockIdx.x * OUTS + o;
	float sum = 0.0f;
	if (idx < count) {
		const float* src = partial + idx;
		int p = grp;
		for (; p + 7 * GROUPS < parts; p += 8 * GROUPS) {
			float v[8];
#pragma unroll
			for (int q = 0; q < 8; q++) v[q] = src[(int64_t)(p + q * GROUPS) * count];
#pragma unroll
			for (int q = 0; q < 8; q++) sum += v[q];
		}
		for (; p < parts; p += GROUPS) sum += src[(int64_t)p * count];
	}
	s[grp][o] = sum;
	__syncthreads();
	if (grp == 0 && idx < count) {
		float tot = 0.0f;
#pragma unroll
		for (int q = 0; q < GROUPS; q++) tot += s[q][o];
		out[idx] = tot;
	}
}

int conv_reduce_partials(const float* partial, int parts, int64_t count, float* out)
{
	if (count <= 4096) conv_reduce_partials_kernel<16><<<dim3((unsigned)ceil_div(count, 16)), dim3(1024), 0, stream()>>>(partial, parts, count, out);
	else conv_reduce_partials_kernel<64><<<dim3((unsigned)ceil_div(count, 64)), dim3(1024), 0, stream()>>>(partial, parts, count, out);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

static bool patch_geometry(const ConvGeo& g)
{
	return g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.kh == 3 && g.kw == 3 && g.pw <= 4 &&
	       (uint64_t)g.Ho * g.Wo <= (1u << 26);  // 32-bit lane offsets in the forward epilogue
}

bool conv_patch_forward_takes(const ConvGeo& g, const float*, const float*)
{
	// below 5 input channels most of an 8-channel chunk would be padding
	return patch_geometry(g) && g.Cin >= 5 && ceil_div((uint64_t)g.Cout, 64) < 65536;
}

template <int BM>
static void launch_patch_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y, bool vec)
{
	typedef PatchFwd<3, 3, BM> P;
	const dim3 grid((unsigned)(ceil_div((uint64_t)g.Wo, P::TW) * ceil_div((uint64_t)g.Ho, P::TH)), (unsigned)ceil_div((uint64_t)g.Cout, P::BM), (unsigned)g.N);
	if (vec) conv2d_patch_forward_kernel<3, 3, BM, true><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y);
	else conv2d_patch_forward_kernel<3, 3, BM, false><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y);
}

int conv_patch_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y)
{
	const bool vec = g.W % 4 == 0 && aligned16(x);
	// 64 output channels per workgroup, or 32 when that leaves fewer padded rows
	if (ceil_div((uint64_t)g.Cout, 32) % 2 == 1) {
		set_kernel_name("conv2d_patch_forward_3x3_32x4x128");
		launch_patch_forward<32>(g, x, w, bias, y, vec);
	} else {
		set_kernel_name("conv2d_patch_forward_3x3_64x4x128");
		launch_patch_forward<64>(g, x, w, bias, y, vec);
	}
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

bool conv_patch_wgrad_takes(const ConvGeo& g)
{
	return patch_geometry(g) && g.Cin >= 9 && ceil_div((uint64_t)g.Cout, 64) < 65536 && ceil_div((uint64_t)g.Cin, 32) < 65536 &&
	       (uint64_t)g.N * g.Ho * ceil_div((uint64_t)g.Wo, 64) < (1ull << 31) &&
	       (uint64_t)g.H * g.W < (1u << 25) && (uint64_t)g.Ho * g.Wo < (1u << 25);  // 32-bit lane offsets over 32 channels
}

// Whether the weight gradient walks chunks of two rows x 32 columns instead of 64 columns of one row: when that wastes
// clearly fewer pixels (a 28-column image: 7/8 of a chunk against 7/16) and the rows allow 16-byte loads.
static bool wgrad_two_row_chunk(const ConvGeo& g, bool vec)
{
	if (!vec || get_option(OPT_CONV_VARIANT) != 0) return false;
	const double wide = (double)g.Wo / (64.0 * (double)ceil_div((uint64_t)g.Wo, 64));
	const double tall = (double)g.Wo / (32.0 * (double)ceil_div((uint64_t)g.Wo, 32)) * (double)g.Ho / (2.0 * (double)ceil_div((uint64_t)g.Ho, 2));
	return tall > 1.15 * wide;
}

static uint64_t wgrad_chunks(const ConvGeo& g, bool two_row)
{
	return two_row ? (uint64_t)g.N * ceil_div((uint64_t)g.Ho, 2) * ceil_div((uint64_t)g.Wo, 32) : (uint64_t)g.N * g.Ho * ceil_div((uint64_t)g.Wo, 64);
}

// upper_bound: the largest count any kernel choice can give (for sizing the workspace, so that a change of the
// tuning option between the size query and the call can never make the kernel write past it)
int conv_patch_wgrad_parts(const ConvGeo& g, bool upper_bound)
{
	typedef PatchWgrad<3, 3> P;
	// two workgroups per CU over all (co block, ci block) pairs, at least four chunks per part
	const uint64_t blocks = ceil_div((uint64_t)g.Cout, P::BM) * ceil_div((uint64_t)g.Cin, P::CIB);
	// one workgroup per CU; two with the unpipelined kernel (rows that do not allow 16-byte loads, or conv_variant 3)
	const bool vec = g.W % 4 == 0 && g.Wo % 4 == 0;
	const uint64_t chunks = upper_bound ? std::max(wgrad_chunks(g, false), wgrad_chunks(g, true)) : wgrad_chunks(g, wgrad_two_row_chunk(g, vec));
	uint64_t parts = std::max<uint64_t>(1, (upper_bound || get_option(OPT_CONV_VARIANT) == 3 || !vec ? 512 : 256) / blocks);
	parts = std::min<uint64_t>(parts, std::max<uint64_t>(1, chunks / 4));
	const uint64_t per = ceil_div(chunks, parts);
	return (int)ceil_div(chunks, per);
}

int conv_patch_wgrad(const ConvGeo& g, const float* x, const float* dy, float* partial, int parts)
{
	typedef PatchWgrad<3, 3> P;
	const bool vec = g.W % 4 == 0 && aligned16(x) && g.Wo % 4 == 0 && aligned16(dy);
	const bool two_row = wgrad_two_row_chunk(g, g.W % 4 == 0 && g.Wo % 4 == 0) && vec;
	const uint64_t chunks = wgrad_chunks(g, two_row);
	const int per = (int)ceil_div(chunks, (uint64_t)parts);
	const dim3 grid((unsigned)parts, (unsigned)ceil_div((uint64_t)g.Cout, P::BM), (unsigned)ceil_div((uint64_t)g.Cin, P::CIB));
	if (two_row) {
		set_kernel_name("conv2d_patch_wgrad_3x3_64x32_2x32");
		conv2d_patch_wgrad_kernel<3, 3, true, true, true><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	if (get_option(OPT_CONV_VARIANT) == 0 && conv_patch_fast_wgrad_takes(g, x, dy)) return conv_patch_fast_wgrad(g, x, dy, partial, parts);
	set_kernel_name("conv2d_patch_wgrad_3x3_64x32");
	if (get_option(OPT_CONV_VARIANT) == 3 || !vec) {
		set_kernel_name("conv2d_patch_wgrad_3x3_64x32_unpipelined");
		if (vec) conv2d_patch_wgrad_kernel<3, 3, true, false><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per);
		else conv2d_patch_wgrad_kernel<3, 3, false, false><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per);
	} else {
		conv2d_patch_wgrad_kernel<3, 3, true, true><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per);
	}
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // namespace lten_hip
