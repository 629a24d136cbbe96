// Conv2d forward, 3x3, stride 1, with the LDS patch filled by direct global->LDS loads.
//
// The same tile and the same MFMA schedule as conv2d_patch_forward_kernel (a workgroup = BM output channels x
// TH rows x 128 columns of one image; TH = 4: wavefront `wave` owns row `wave`, TH = 2: row wave % 2, columns
// 64 (wave / 2) .. + 63; input channels in chunks of four, step
// (cp, i, j) multiplies tap (i, j) of channels 2cp (lanes 0-31) and 2cp + 1 (lanes 32-63)), but a chunk reaches
// LDS without passing through registers: two LDS stages, chunk c + 1 lands in one while chunk c is multiplied
// from the other, one barrier per chunk.
//
// A stage holds the patch [4 channels][TH + 2 rows][136 columns] (column q = input column w0 - 4 + q) and the weights
// [BM channels][36] exactly as they lie in memory, so both are filled by wave-wide loads whose lane L writes 16
// bytes at 16 L: patch float4 number idx is (channel idx / (34 (TH + 2)), row (idx / 34) % (TH + 2), columns 4 (idx % 34) ..);
// weight float4 number idx is (channel idx / 9, floats 4 (idx % 9) ..).  Whether a float4 lies inside the image
// (or names an existing output channel) does not depend on the chunk: lanes whose float4 does not exist never
// load, and their LDS slots keep the zeros written once before the first chunk.  That is the zero padding.
//
// Needs Cin % 4 == 0 (whole chunks, 16-byte aligned weight rows), W % 4 == 0 and 16-byte aligned x and w.
#include "conv_common.h"
#include "gemm_f32_core.h"
#include "lds_async.h"

namespace lten_hip {

namespace {

// VERT: the tile for narrow images, 16 rows x 32 columns: a wavefront owns four rows of 32 pixels (its four MFMA column
// blocks lie below one another instead of side by side), the patch is [4 channels][18 rows][40 columns].  On a 28 x 28
// image 77 % of such tiles are pixels that exist, against 22 % of the 128-column tiles.
// ELEM (with VERT): the patch is fetched four bytes per lane instead of sixteen, for input rows that do not start on
// 16-byte boundaries (a width that is no multiple of four): four times the load instructions, the same bytes.
template <int BM_, int TH_, bool VERT_ = false, bool ELEM_ = false>
struct FastFwd {
	static_assert(TH_ == 4 || TH_ == 2, "a wavefront owns a whole row of the tile (TH = 4) or half a row (TH = 2)");
	static constexpr bool VERT = VERT_, ELEM = ELEM_;
	static_assert(!ELEM || VERT, "the 4-byte patch loads exist for the narrow-image tile");
	static constexpr int BM = BM_, MT = BM / 32, TH = TH_, NT = VERT ? 4 : TH, CB = 4;
	static constexpr int TW = VERT ? 32 : 128, TROWS = VERT ? 16 : TH, PR = TROWS + 2, PWS = TW + 8, F4R = PWS / 4;
	static constexpr int BLOCK_STEP = VERT ? PWS : 32;            // floats between a wavefront's MFMA column blocks in the patch
	static constexpr int PATCH_F4 = CB * PR * F4R;                 // 816
	static constexpr int PATCH_UNITS = ELEM ? 4 * PATCH_F4 : PATCH_F4;  // what a lane fetches: a float or four
	static constexpr int PATCH_LOAD_BYTES = ELEM ? 256 : 1024;          // bytes of one wave-wide patch load
	static constexpr int PATCH_LOADS = (PATCH_UNITS + 63) / 64;    // 13 (45 with ELEM)
	static constexpr int PATCH_BYTES = PATCH_LOADS * PATCH_LOAD_BYTES;
	static constexpr int W_F4 = BM * 9;                            // 36 floats per channel
	static constexpr int W_LOADS = (W_F4 + 63) / 64;
	static constexpr int W_BYTES = W_LOADS * 1024;
	static constexpr int STAGE = PATCH_BYTES + W_BYTES;
	static constexpr int LOADS = PATCH_LOADS + W_LOADS;
	static constexpr int LPW = (LOADS + 3) / 4;                    // per wavefront, the last ones may not exist
	static constexpr int STEPS = (CB / 2) * 9;                     // 18 MFMA steps per chunk
	static constexpr int NR = MT + NT, NM = MT * NT;
};

}  // namespace

template <int BM, int TH, bool VERT = false, bool ELEM = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(BM * TH == 256 ? 2 : 4, BM * TH == 256 ? 2 : 4))) void conv2d_patch_fast_forward_kernel(
    ConvGeo g, const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ y)
{
	typedef FastFwd<BM, TH, VERT, ELEM> P;
	__shared__ __attribute__((aligned(1024))) uint8_t smem[2 * P::STAGE];

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int lrow = lane & 31, half = lane >> 5;
	// this wavefront's (first) row and first column in the tile
	const int wrow = VERT ? 4 * wave : (TH == 4 ? wave : (wave & 1)), wcol = (VERT || TH == 4) ? 0 : (wave >> 1) * 64;
	const int tiles_w = (g.Wo + P::TW - 1) / P::TW;
	const int w0 = (int)(blockIdx.x % tiles_w) * P::TW, h0 = (int)(blockIdx.x / tiles_w) * P::TROWS;
	const int co0 = blockIdx.y * BM, n = blockIdx.z;
	const int Kc = g.Cin * 9;
	const float* xn = x + (int64_t)n * g.Cin * g.H * g.W;
	const float* wb = w + (int64_t)co0 * Kc;

	// ---- what this lane fetches for each of its wavefront's loads (load q = wave + 4 i)
	uint32_t voff[P::LPW], slot[P::LPW];
	bool valid[P::LPW];
	const uint32_t smem_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
#pragma unroll
	for (int i = 0; i < P::LPW; i++) {
		const int q = wave + 4 * i;
		valid[i] = false;
		voff[i] = 0;
		slot[i] = smem_addr + (q < P::PATCH_LOADS ? q * P::PATCH_LOAD_BYTES : P::PATCH_BYTES + (q - P::PATCH_LOADS) * 1024);
		if (q < P::PATCH_LOADS) {
			const int idx = q * 64 + lane;
			constexpr int UPR = ELEM ? P::PWS : P::F4R;  // units per patch row
			const int f = idx % UPR, r = (idx / UPR) % P::PR, c = idx / (UPR * P::PR);
			const int gy = h0 - g.ph + r, gx = w0 - 4 + (ELEM ? f : 4 * f);
			if (idx < P::PATCH_UNITS && gy >= 0 && gy < g.H && gx >= 0 && gx < g.W) {
				valid[i] = true;
				voff[i] = (uint32_t)(((c * g.H + gy) * g.W + gx) * 4);
			}
		} else if (q < P::LOADS) {
			const int idx = (q - P::PATCH_LOADS) * 64 + lane;
			const int f = idx % 9, co = idx / 9;
			if (idx < P::W_F4 && co0 + co < g.Cout) {
				valid[i] = true;
				voff[i] = (uint32_t)((co * Kc + 4 * f) * 4);
			}
		}
	}
	const int64_t x_step = (int64_t)P::CB * g.H * g.W;
	auto load_one = [&](int i, int stage, int kt) {
		if (wave + 4 * i >= P::LOADS) return;  // the same for the whole wavefront
		const float* base = wave + 4 * i < P::PATCH_LOADS ? xn + kt * x_step : wb + kt * (P::CB * 9);
		if (valid[i]) {
			if (ELEM && wave + 4 * i < P::PATCH_LOADS) async_load4(slot[i] + stage * P::STAGE, base, voff[i]);
			else async_load16(slot[i] + stage * P::STAGE, base, voff[i]);
		}
	};

	// ---- zeros everywhere once: what no load ever writes is the padding
	for (int i = tid; i < 2 * P::STAGE / 16; i += 256) reinterpret_cast<float4*>(smem)[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
	__syncthreads();

	const int KT = g.Cin / P::CB;
#pragma unroll
	for (int i = 0; i < P::LPW; i++) load_one(i, 0, 0);
	if (KT > 1) {
#pragma unroll
		for (int i = 0; i < P::LPW; i++) load_one(i, 1, 1);
	}

	// ---- operand addresses: a per-lane base plus immediates
	const int off_a = P::PATCH_BYTES + (lrow * 36 + half * 9) * 4;
	const int off_b = ((half * P::PR + wrow) * P::PWS + wcol + lrow + 4 - g.pw) * 4;
	auto read_one = [&](float (&fa)[P::MT], float (&fb)[P::NT], const uint8_t* sbase, int s, int e) {
		const int cp = s / 9, tap = s % 9, ti = tap / 3, tj = tap % 3;
		if (e < P::MT) fa[e] = *reinterpret_cast<const float*>(sbase + off_a + (e * 32 * 36 + 2 * cp * 9 + tap) * 4);
		else fb[e - P::MT] = *reinterpret_cast<const float*>(sbase + off_b + ((2 * cp * P::PR + ti) * P::PWS + tj + (e - P::MT) * P::BLOCK_STEP) * 4);
	};

	v16f acc[P::MT][P::NT];
#pragma unroll
	for (int m = 0; m < P::MT; m++)
#pragma unroll
		for (int t = 0; t < P::NT; t++)
#pragma unroll
			for (int r = 0; r < 16; r++) acc[m][t][r] = 0.0f;

	// One step in the exact instruction order wanted: its MFMAs and, behind them, the LDS reads of the next step's
	// operands and (in the step after the barrier) this wavefront's loads of the chunk after next.
	auto beat = [&](const float (&ca)[P::MT], const float (&cb)[P::NT], float (&na)[P::MT], float (&nb)[P::NT], int stg, int s, bool read_next,
	                bool refill, int refill_stage, int refill_kt) {
		const uint8_t* sbase = smem + stg * P::STAGE;
#pragma unroll
		for (int m = 0; m < P::NM; m++) {
			acc[m / P::NT][m % P::NT] = __builtin_amdgcn_mfma_f32_32x32x2f32(ca[m / P::NT], cb[m % P::NT], acc[m / P::NT][m % P::NT], 0, 0, 0);
			if (read_next) {
#pragma unroll
				for (int e = m; e < P::NR; e += P::NM) read_one(na, nb, sbase, s, e);
			}
			if (refill) {
#pragma unroll
				for (int l = m; l < P::LPW; l += P::NM) load_one(l, refill_stage, refill_kt);
			}
			__builtin_amdgcn_sched_barrier(0);
		}
	};

	float fa0[P::MT], fb0[P::NT], fa1[P::MT], fb1[P::NT];
	// Only the first chunk has to be there: every workgroup of the chip asks for its first two chunks at the same moment
	// (38 MB at config 5's second layer), and waiting for both kept the matrix pipe idle twice as long.  Loads complete
	// in order, so chunk 0 has landed once no more loads are out than were issued for chunk 1 (a load none of whose
	// lanes takes part is not issued, hence the count).
	int behind = 0;
	if (KT > 1) {
#pragma unroll
		for (int i = 0; i < P::LPW; i++)
			if (wave + 4 * i < P::LOADS && __ballot(valid[i]) != 0) behind++;
	}
	switch (behind) {
	case 0: wait_vmcnt_lgkm0<0>(); break;
	case 1: wait_vmcnt_lgkm0<1>(); break;
	case 2: wait_vmcnt_lgkm0<2>(); break;
	case 3: wait_vmcnt_lgkm0<3>(); break;
	case 4: wait_vmcnt_lgkm0<4>(); break;
	case 5: wait_vmcnt_lgkm0<5>(); break;
	case 6: wait_vmcnt_lgkm0<6>(); break;
	case 7: wait_vmcnt_lgkm0<7>(); break;
	case 8: wait_vmcnt_lgkm0<8>(); break;
	case 9: wait_vmcnt_lgkm0<9>(); break;
	case 10: wait_vmcnt_lgkm0<10>(); break;
	case 11: wait_vmcnt_lgkm0<11>(); break;
	case 12: wait_vmcnt_lgkm0<12>(); break;
	case 13: wait_vmcnt_lgkm0<13>(); break;
	case 14: wait_vmcnt_lgkm0<14>(); break;
	default: wait_vmcnt_lgkm0<0>(); break;
	}
	__syncthreads();
#pragma unroll
	for (int e = 0; e < P::NR; e++) read_one(fa0, fb0, smem, 0, e);

	auto inner_beats = [&](int stg) {
#pragma unroll
		for (int s = 0; s + 1 < P::STEPS; s++) {
			if (s & 1) beat(fa1, fb1, fa0, fb0, stg, s + 1, true, false, 0, 0);
			else beat(fa0, fb0, fa1, fb1, stg, s + 1, true, false, 0, 0);
		}
	};
	int stage = 0, kt = 0;
	for (; kt + 2 < KT; kt++) {
		inner_beats(stage);
		wait_vmcnt_lgkm0<0>();  // own loads of chunk kt + 1 have landed, own reads of chunk kt are done
		__syncthreads();
		// STEPS is even: the last step's operands sit in set 1; the stage just read is refilled with chunk kt + 2
		beat(fa1, fb1, fa0, fb0, stage ^ 1, 0, true, true, stage, kt + 2);
		stage ^= 1;
	}
	if (kt + 1 < KT) {  // the last but one chunk: nothing left to load
		inner_beats(stage);
		wait_vmcnt_lgkm0<0>();
		__syncthreads();
		beat(fa1, fb1, fa0, fb0, stage ^ 1, 0, true, false, 0, 0);
		stage ^= 1;
	}
	inner_beats(stage);
	beat(fa1, fb1, fa0, fb0, stage, 0, false, false, 0, 0);

	// Epilogue: all bias values first, then stores whose address is a shared part plus a lane offset.
	const int ho = h0 + wrow;
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
	float* yw = y + (((int64_t)n * g.Cout + co0) * g.Ho + ho) * g.Wo + w0 + wcol;
	const unsigned y_lane = (unsigned)(half * 4 * plane) + lrow;
	const unsigned y_step = VERT ? (unsigned)g.Wo : 32u;  // from one of the wavefront's column blocks to the next: a row down, or 32 columns on
	if (co0 + BM <= g.Cout && w0 + P::TW <= g.Wo && (!VERT || h0 + P::TROWS <= g.Ho)) {
#pragma unroll
		for (int m = 0; m < P::MT; m++)
#pragma unroll
			for (int r = 0; r < 16; r++) {
				float* yr = yw + (m * 32 + (r >> 2) * 8 + (r & 3)) * plane;
#pragma unroll
				for (int t = 0; t < P::NT; t++) __builtin_nontemporal_store(acc[m][t][r] + bv[m][r], &yr[y_lane + t * y_step]);  // y is written once and not read here
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
			for (int t = 0; t < P::NT; t++) {
				const bool inside = VERT ? (ho + t < g.Ho && w0 + lrow < g.Wo) : (w0 + wcol + t * 32 + lrow < g.Wo);
				if (inside) __builtin_nontemporal_store(acc[m][t][r] + bv[m][r], &yr[y_lane + t * y_step]);
			}
		}
}

bool conv_patch_fast_forward_vertical(const ConvGeo& g);

bool conv_patch_fast_forward_takes(const ConvGeo& g, const float* x, const float* w)
{
	// Rows off 16-byte boundaries: the narrow-image tile has a form with 4-byte patch loads, the 128-column tile has not.
	// The narrow-image tiles need enough workgroups: with few, the implicit GEMM over the batch's flattened pixels is
	// ahead (8 x 128 x 28 x 28 -> 128 channels, 64 workgroups: 55 against 72 us; 64 x 32 x 28 x 28 -> 64, 256 workgroups:
	// 44 against 23 us), and the 4-byte form, whose loads are four times as many, needs more of them (32 x 32 x 30 x 30
	// -> 64, 128 workgroups: 24 against 31 us; 32 x 48 x 50 x 50 -> 96, 768 workgroups: 154 against 95 us).
	const bool rows16 = g.W % 4 == 0 && aligned16(x);
	if (conv_patch_fast_forward_vertical(g)) {
		const uint64_t tiles = ceil_div((uint64_t)g.Wo, 32) * ceil_div((uint64_t)g.Ho, 16), wgs = tiles * ceil_div((uint64_t)g.Cout, 32) * g.N;
		// ... and images that fill at least half of their tiles (64 x 256 x 7 x 7 -> 256 fills a tenth: 118 against 307 us)
		const bool half_full = 2 * (uint64_t)g.Ho * g.Wo >= tiles * 16 * 32;
		if ((wgs < (rows16 ? 200u : 256u) || !half_full) && get_option(OPT_CONV_VARIANT) == 0) return false;
	}
	return g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.kh == 3 && g.kw == 3 && g.pw <= 4 && g.Cin % 4 == 0 && g.Cin >= 8 &&
	       (rows16 || (conv_patch_fast_forward_vertical(g) && get_option(OPT_CONV_VARIANT) != 5)) && aligned16(w) && (uint64_t)g.H * g.W < (1u << 26) && (uint64_t)g.Ho * g.Wo <= (1u << 26) &&
	       (uint64_t)64 * g.Cin * 9 * 4 < (1ull << 31) && ceil_div((uint64_t)g.Cout, 32) < 65536 && g.N < 65536;
}

// Images of at most 96 output columns take the 16 x 32 tiles (a quarter or more of a 128-column tile would be padding;
// measured equal at 100 to 112 columns, ahead below: 16 x 64 x 64 x 64 -> 64 channels 77 -> 39 us, 64 x 32 x 28 x 28 -> 64: 61 -> 23 us).
bool conv_patch_fast_forward_vertical(const ConvGeo& g) { return g.Wo <= 96; }

int conv_patch_fast_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y)
{
	const unsigned blocks64 = (unsigned)ceil_div((uint64_t)g.Cout, 64), blocks32 = (unsigned)ceil_div((uint64_t)g.Cout, 32);
	if (conv_patch_fast_forward_vertical(g) && get_option(OPT_CONV_VARIANT) != 5) {
		const unsigned vtiles = (unsigned)(ceil_div((uint64_t)g.Wo, 32) * ceil_div((uint64_t)g.Ho, 16));
		// 64 output channels per workgroup when that still gives every CU two workgroups, else 32
		const bool elem = g.W % 4 != 0 || !aligned16(x);  // 4-byte patch loads
		if (blocks32 % 2 == 0 && (uint64_t)vtiles * blocks64 * g.N >= 512) {
			set_kernel_name(elem ? "conv2d_patch_fast_forward_3x3_64x16x32_e4" : "conv2d_patch_fast_forward_3x3_64x16x32");
			if (elem) conv2d_patch_fast_forward_kernel<64, 4, true, true><<<dim3(vtiles, blocks64, (unsigned)g.N), dim3(256), 0, stream()>>>(g, x, w, bias, y);
			else conv2d_patch_fast_forward_kernel<64, 4, true><<<dim3(vtiles, blocks64, (unsigned)g.N), dim3(256), 0, stream()>>>(g, x, w, bias, y);
		} else {
			set_kernel_name(elem ? "conv2d_patch_fast_forward_3x3_32x16x32_e4" : "conv2d_patch_fast_forward_3x3_32x16x32");
			if (elem) conv2d_patch_fast_forward_kernel<32, 4, true, true><<<dim3(vtiles, blocks32, (unsigned)g.N), dim3(256), 0, stream()>>>(g, x, w, bias, y);
			else conv2d_patch_fast_forward_kernel<32, 4, true><<<dim3(vtiles, blocks32, (unsigned)g.N), dim3(256), 0, stream()>>>(g, x, w, bias, y);
		}
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	const unsigned tiles_w = (unsigned)ceil_div((uint64_t)g.Wo, 128);
	const unsigned tiles = tiles_w * (unsigned)ceil_div((uint64_t)g.Ho, 4);
	if (blocks32 % 2 == 1) {
		set_kernel_name("conv2d_patch_fast_forward_3x3_32x4x128");
		conv2d_patch_fast_forward_kernel<32, 4><<<dim3(tiles, blocks32, (unsigned)g.N), dim3(256), 0, stream()>>>(g, x, w, bias, y);
	} else if ((uint64_t)tiles * blocks64 * g.N < 2048 && get_option(OPT_CONV_VARIANT) != 5) {
		// Few workgroups per CU slot (two at a time fit): all of them reach their store epilogue together and the
		// matrix pipe waits while y is written.  Tiles of two rows double the workgroups and fit four to a CU, so
		// one workgroup's stores overlap another's MFMAs (config 5 layer 2: 192 -> 178 us on the same box); with
		// many rounds of workgroups the taller tile's smaller halo wins.  conv_variant 5 keeps the taller tile.
		set_kernel_name("conv2d_patch_fast_forward_3x3_64x2x128");
		const unsigned tiles2 = tiles_w * (unsigned)ceil_div((uint64_t)g.Ho, 2);
		conv2d_patch_fast_forward_kernel<64, 2><<<dim3(tiles2, blocks64, (unsigned)g.N), dim3(256), 0, stream()>>>(g, x, w, bias, y);
	} else {
		set_kernel_name("conv2d_patch_fast_forward_3x3_64x4x128");
		conv2d_patch_fast_forward_kernel<64, 4><<<dim3(tiles, blocks64, (unsigned)g.N), dim3(256), 0, stream()>>>(g, x, w, bias, y);
	}
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // namespace lten_hip
