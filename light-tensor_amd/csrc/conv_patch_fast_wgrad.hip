// Conv2d weight gradient, 3x3, stride 1, padding 1, with both LDS tiles filled by direct global->LDS loads.
//
// The same tile and MFMA schedule as conv2d_patch_wgrad_kernel (rows = 64 output channels, columns = (tap, 32
// input channels), reduction over pixels in chunks of 64 pixels of one output row; wavefront (row tile mt, pixel
// half) holds the nine tap tiles), one workgroup per CU, two LDS stages, one barrier per chunk.  What differs is
// how a chunk reaches LDS: no registers, no LDS stores, no branches and little vector ALU work on the way.
// Measured on this part, for a wavefront that is alone on its SIMD: a vector ALU instruction between two fp32
// MFMAs delays the second one by about 12 shader clocks (4 for every further one), a taken branch by far more,
// while LDS reads and scalar instructions (a dozen per MFMA) cost nothing.  The register-staged kernel spends 12 %
// of its cycles fetching and 4 % on the staging stores; this one keeps the matrix pipe about 90 % busy.
//
// A wave-wide direct load writes lane L's 16 bytes at LDS address base + 16 L, so the LDS layout is fixed by
// which global float4 each lane fetches:
//   dy tile   load j = 4 fg + cg (fg = group of four pixel quads, cg = group of 16 channels): lane L = 16 fq + cq
//             fetches pixels 4 (4 fg + fq) .. + 3 of channel 16 cg + cq: 16 rows x 64 contiguous bytes per load
//   patch     [32 channels][3 rows][18 float4] with a channel pitch of 55 float4; float4 number c = 64 j + L of
//             load j is (channel c / 55, row (c % 55) / 18, input columns w0 - 4 + 4 ((c % 55) % 18) ..)
// With 16-byte granules the 32 lanes of an operand read (32 channels, one pixel) cannot all fall on different
// banks (several lanes per bank with any pitch); the reads are issued nine MFMAs ahead and the loop without its
// loads still runs at 97 % of the MFMA rate, so that does not matter here.
// Lanes whose float4 never exists (pad slot, channel beyond Cin or Cout) never load; their slots keep the zeros
// written once.  Lanes whose float4 lies outside the image in this chunk only (halo row above the first / below
// the last image row, halo float4 left of the first / right of the last column) store zeros instead of loading.
// Both are done by setting the execution mask, not by branching.
//
// Needs W % 64 == 0 (whole chunks; the halo float4s are then inside or outside the image as a whole) and 16-byte
// aligned x and dy.
#include <type_traits>

#include "conv_common.h"
#include "gemm_f32_core.h"
#include "lds_async.h"

namespace lten_hip {

namespace {

struct FastWgrad {
	static constexpr int BM = 64, CIB = 32, TW = 64, TAPS = 9, STEPS = TW / 4, SLOTS = STEPS * TAPS;
	static constexpr int DY_LOADS = 16, DY_BYTES = DY_LOADS * 1024;
	static constexpr int F4_ROW = 18, PITCH_F4 = 55, PWS = F4_ROW * 4, CS = PITCH_F4 * 4;
	static constexpr int PATCH_F4 = CIB * PITCH_F4;             // 1760
	static constexpr int PATCH_LOADS = (PATCH_F4 + 63) / 64;    // 28
	static constexpr int PATCH_BYTES = PATCH_LOADS * 1024;
	static constexpr int STAGE = DY_BYTES + PATCH_BYTES;        // 45056
	static constexpr int DPW = DY_LOADS / 4, PPW = PATCH_LOADS / 4;  // loads per wavefront
	static constexpr int TAPS_PER_ROUND = 2 * STAGE / 4 / (2 * 64 * 16);  // taps whose accumulators fit the final exchange
	static_assert(PATCH_LOADS % 4 == 0 && TAPS_PER_ROUND >= 1, "tile shape");
	// chunk flags: why a float4 does not exist in this chunk
	static constexpr unsigned TOP = 1, BOTTOM = 2, LEFT = 4, RIGHT = 8;
};

}  // namespace

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void conv2d_patch_fast_wgrad_kernel(
    ConvGeo g, const float* __restrict__ x, const float* __restrict__ dy, float* __restrict__ partial, int chunks_per_part)
{
	typedef FastWgrad P;
	__shared__ __attribute__((aligned(1024))) uint8_t smem[2 * P::STAGE];

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int lrow = lane & 31, half = lane >> 5;
	const int mt = wave & 1, phalf = wave >> 1;
	const int co0 = blockIdx.y * P::BM, ci0 = blockIdx.z * P::CIB;
	const int tiles_w = g.W / P::TW;
	const int total = g.N * g.H * tiles_w;
	const int begin = blockIdx.x * chunks_per_part, end = min(total, begin + chunks_per_part);
	const int64_t plane = (int64_t)g.H * g.W;
	const uint32_t smem_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
	const uint32_t lane16 = lane * 16;
	const lds_v4f zero4 = {0.0f, 0.0f, 0.0f, 0.0f};

	// ---- what this lane fetches: dy loads j = 4 wave + i, patch loads j = wave + 4 i
	const int cq = lane & 15, fq = lane >> 4;
	const uint32_t dy_voff = (uint32_t)((cq * plane + 4 * (4 * wave + fq)) * 4);  // + i * 16 channels, in the base
	// which lanes take part is kept as execution masks (wave-wide bit sets in scalar registers)
	uint64_t dy_mask[P::DPW], p_exists[P::PPW];
#pragma unroll
	for (int i = 0; i < P::DPW; i++) dy_mask[i] = __ballot(co0 + 16 * i + cq < g.Cout);
	uint32_t p_voff[P::PPW], p_flags[P::PPW];
#pragma unroll
	for (int i = 0; i < P::PPW; i++) {
		const int c = (wave + 4 * i) * 64 + lane;
		const int ci = c / P::PITCH_F4, rem = c % P::PITCH_F4, r = rem / P::F4_ROW, f = rem % P::F4_ROW;
		const bool never = rem == P::PITCH_F4 - 1 || ci >= P::CIB || ci0 + ci >= g.Cin;
		p_flags[i] = never ? 0 : (r == 0 ? P::TOP : 0) | (r == 2 ? P::BOTTOM : 0) | (f == 0 ? P::LEFT : 0) | (f == P::F4_ROW - 1 ? P::RIGHT : 0);
		p_exists[i] = __ballot(!never);
		p_voff[i] = never ? 0 : (uint32_t)((((int64_t)ci * g.H + r) * g.W + 4 * f) * 4);  // from (row ho - 1, column w0 - 4) of channel ci0
	}
	// The chunk's position is kept as two byte addresses that advance with it: dyb = (image, channel co0, row ho,
	// column w0) of dy, xb = (image, channel ci0, row ho - 1, column w0 - 4) of x (which may lie before the array;
	// lanes that would read there are masked).  Rows follow each other in memory, so the next chunk is 256 bytes
	// on, except after the last row of an image, where the remaining channels of that image are skipped.
	int ho_c = (begin / tiles_w) % g.H, w0_c = (begin % tiles_w) * P::TW;
	const int n_first = begin / (tiles_w * g.H);
	const char* dyb = reinterpret_cast<const char*>(dy + (((int64_t)n_first * g.Cout + co0) * g.H + ho_c) * g.W + w0_c);
	const char* xb = reinterpret_cast<const char*>(x + (((int64_t)n_first * g.Cin + ci0) * g.H + ho_c - 1) * g.W + w0_c - 4);
	const int64_t dy_image_skip = (int64_t)(g.Cout - 1) * plane * 4, x_image_skip = (int64_t)(g.Cin - 1) * plane * 4;
	const int64_t dy_group_step = 16 * plane * 4;  // 16 channels on
	auto next_chunk = [&]() {
		w0_c += P::TW;
		dyb += P::TW * 4;
		xb += P::TW * 4;
		if (w0_c >= g.W) {
			w0_c = 0;
			if (++ho_c == g.H) {
				ho_c = 0;
				dyb += dy_image_skip;
				xb += x_image_skip;
			}
		}
	};
	// one load of the chunk at (dyb, xb, ho_c, w0_c) into `stage`: k < DPW is a dy load, the others are patch loads
	auto load_piece = [&](int stage, int k) {
		const uint32_t stage_addr = smem_addr + stage * P::STAGE;
		if (k < P::DPW) {
			async_load16_masked(dy_mask[k], stage_addr + (4 * wave + k) * 1024, dyb + k * dy_group_step, dy_voff);
			return;
		}
		const int i = k - P::DPW;
		const unsigned cf = (ho_c == 0 ? P::TOP : 0) | (ho_c == g.H - 1 ? P::BOTTOM : 0) | (w0_c == 0 ? P::LEFT : 0) |
		                    (w0_c + P::TW >= g.W ? P::RIGHT : 0);
		const uint64_t outside = __ballot((p_flags[i] & cf) != 0);
		const uint32_t slot = stage_addr + P::DY_BYTES + (wave + 4 * i) * 1024;
		async_load16_masked(p_exists[i] & ~outside, slot, xb, p_voff[i]);
		lds_zero16_masked(outside, slot + lane16, zero4);
	};
	constexpr int PIECES = P::DPW + P::PPW;

	// ---- zeros everywhere once, then the first chunk
	for (int i = tid; i < 2 * P::STAGE / 16; i += 256) reinterpret_cast<float4*>(smem)[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
	__syncthreads();
	if (begin < end) {
#pragma unroll
		for (int k = 0; k < PIECES; k++) load_piece(0, k);
		next_chunk();
	}

	v16f acc[P::TAPS];
#pragma unroll
	for (int t = 0; t < P::TAPS; t++)
#pragma unroll
		for (int r = 0; r < 16; r++) acc[t][r] = 0.0f;

	// operand addresses: a per-lane base plus immediates
	const int off_a = ((phalf * 8 + mt * 2 + (lrow >> 4)) * 1024) + (lrow & 15) * 16 + half * 4;
	const int off_b = P::DY_BYTES + (lrow * P::CS + phalf * (P::TW / 2) + half + 3) * 4;

	wait_vmcnt_lgkm0<0>();
	__syncthreads();

	// MORE: a chunk follows (at (n_c, ho_c, w0_c)), whose loads go out behind the first MFMAs into the other stage
	auto run_chunk = [&](int cur, auto more_tag) {
		constexpr bool MORE = decltype(more_tag)::value;
		const uint8_t* sa = smem + cur * P::STAGE + off_a;
		const uint8_t* sb = smem + cur * P::STAGE + off_b;
		float fa[2], fb[2][P::TAPS];
		auto read_a = [&](int s) { fa[s & 1] = *reinterpret_cast<const float*>(sa + (s / 8) * 4096 + ((s / 2) % 4) * 256 + (s % 2) * 8); };
		auto read_b = [&](int s, int t) { fb[s & 1][t] = *reinterpret_cast<const float*>(sb + ((t / 3) * P::PWS + (t % 3) + 2 * s) * 4); };
		read_a(0);
#pragma unroll
		for (int t = 0; t < P::TAPS; t++) read_b(0, t);
#pragma unroll
		for (int s = 0; s < P::STEPS; s++) {
#pragma unroll
			for (int t = 0; t < P::TAPS; t++) {
				acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s & 1], fb[s & 1][t], acc[t], 0, 0, 0);
				if (s + 1 < P::STEPS) {
					if (t == 0) read_a(s + 1);
					read_b(s + 1, t);
				}
				const int k = s * P::TAPS + t;
				if (MORE && k < PIECES) load_piece(cur ^ 1, k);
				__builtin_amdgcn_sched_barrier(0);
			}
		}
		if (MORE) next_chunk();
		wait_vmcnt_lgkm0<0>();  // own loads of the next chunk have landed, own reads of this one are done
		__syncthreads();
	};
	int cur = 0;
	for (int chunk = begin; chunk + 1 < end; chunk++) {
		run_chunk(cur, std::true_type{});
		cur ^= 1;
	}
	if (begin < end) run_chunk(cur, std::false_type{});

	// pixel half 1 hands its sums to pixel half 0 of the same row tile, TAPS_PER_ROUND taps at a time
	float* lds = reinterpret_cast<float*>(smem);
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

bool conv_patch_fast_wgrad_takes(const ConvGeo& g, const float* x, const float* dy)
{
	return g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.kh == 3 && g.kw == 3 && g.ph == 1 && g.pw == 1 && g.W % 64 == 0 &&
	       aligned16(x) && aligned16(dy) && (uint64_t)(g.H + 2) * g.W < (1u << 24);  // lane offsets of up to 32 channel planes fit 32 bits
}

int conv_patch_fast_wgrad(const ConvGeo& g, const float* x, const float* dy, float* partial, int parts)
{
	typedef FastWgrad P;
	const uint64_t chunks = (uint64_t)g.N * g.H * (g.W / P::TW);
	const int per = (int)ceil_div(chunks, (uint64_t)parts);
	const dim3 grid((unsigned)parts, (unsigned)ceil_div((uint64_t)g.Cout, P::BM), (unsigned)ceil_div((uint64_t)g.Cin, P::CIB));
	set_kernel_name("conv2d_patch_fast_wgrad_3x3_64x32");
	conv2d_patch_fast_wgrad_kernel<<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // namespace lten_hip
