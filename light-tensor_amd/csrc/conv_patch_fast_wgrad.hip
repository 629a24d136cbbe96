// Conv2d weight gradient, 3x3, stride 1, padding 1, with both LDS tiles filled by direct global->LDS loads and every
// input row fetched once per column strip.
//
// The same tile and MFMA schedule as conv2d_patch_wgrad_kernel (rows = 64 output channels, columns = (tap, 32
// input channels), reduction over pixels in chunks of 64 pixels of one output row; wavefront (row tile mt, pixel
// half) holds the nine tap tiles), one workgroup per CU, one barrier per chunk.  What differs is how a chunk
// reaches LDS: no registers, no LDS stores, no branches and little vector ALU work on the way.
// Measured on this part, for a wavefront that is alone on its SIMD: a vector ALU instruction between two fp32
// MFMAs delays the second one by about 12 shader clocks (4 for every further one), a taken branch by far more,
// while LDS reads and scalar instructions (a dozen per MFMA) cost nothing.
//
// Chunks are walked down a strip of 64 columns: (image, strip, row) with the row running fastest.  Output row ho
// needs input rows ho - 1 .. ho + 1, of which the chunk before it (row ho - 1) already had two, so the input rows
// live in a ring of eight LDS slots and a chunk fetches one new row (a third of the patch).  Only the first chunk of
// a workgroup and the first row of a strip fetch all three.  A ring slot holds [32 channels][19 float4]: float4 f
// of a channel is input columns w0 - 4 + 4 f .. + 3 (f = 0 and f = 17 are the halo, f = 18 is padding that keeps
// the 32 channels of an operand read on eight banks).
//
// A wave-wide direct load writes lane L's 16 bytes at LDS address base + 16 L, so the LDS layout is fixed by
// which global float4 each lane fetches:
//   dy tile   load j = 4 fg + cg (fg = group of four pixel quads, cg = group of 16 channels): lane L = 16 fq + cq
//             fetches pixels 4 (4 fg + fq) .. + 3 of channel 16 cg + cq: 16 rows x 64 contiguous bytes per load
//   row       float4 number c = 64 j + L of load j is (channel c / 19, float4 c % 19)
// Lanes whose float4 never exists (pad slot, channel beyond Cin or Cout) never load.  Lanes whose float4 lies
// outside the image (a whole row above the first / below the last image row, the halo float4 left of the first /
// right of the last column) store zeros instead of loading.  Both are done by setting the execution mask, not by
// branching.
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
	static constexpr int BM = 64, CIB = 32, TW = 64, TAPS = 9, STEPS = TW / 4;
	static constexpr int DY_LOADS = 16, DY_BYTES = DY_LOADS * 1024, DPW = DY_LOADS / 4;
	static constexpr int F4_ROW = 18, PITCH_F4 = 19, CS = PITCH_F4 * 4;
	static constexpr int ROW_F4 = CIB * PITCH_F4;               // 608
	static constexpr int ROW_LOADS = (ROW_F4 + 63) / 64;        // 10
	static constexpr int ROW_BYTES = ROW_LOADS * 1024;
	static constexpr int RPW = (ROW_LOADS + 3) / 4;             // row loads per wavefront; the last may not exist
	static constexpr int RING = 8, RING0 = 2 * DY_BYTES;        // two dy stages, then the ring
	static constexpr int TOTAL = RING0 + RING * ROW_BYTES;      // 114688
	static_assert(TOTAL / 4 >= 2 * 64 * 16 * TAPS, "the final exchange of the nine tap tiles fits LDS in one round");
};

}  // namespace

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void conv2d_patch_fast_wgrad_kernel(
    ConvGeo g, const float* __restrict__ x, const float* __restrict__ dy, float* __restrict__ partial, int chunks_per_part)
{
	typedef FastWgrad P;
	__shared__ __attribute__((aligned(1024))) uint8_t smem[P::TOTAL];

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

	// ---- what this lane fetches: dy loads j = 4 wave + i, row loads j = wave + 4 i
	const int cq = lane & 15, fq = lane >> 4;
	const uint32_t dy_voff = (uint32_t)((cq * plane + 4 * (4 * wave + fq)) * 4);  // + i * 16 channels, in the base
	// which lanes take part is kept as execution masks (wave-wide bit sets in scalar registers)
	uint64_t dy_mask[P::DPW], r_exists[P::RPW], r_left[P::RPW], r_right[P::RPW];
#pragma unroll
	for (int i = 0; i < P::DPW; i++) dy_mask[i] = __ballot(co0 + 16 * i + cq < g.Cout);
	uint32_t r_voff[P::RPW];
#pragma unroll
	for (int i = 0; i < P::RPW; i++) {
		const int j = wave + 4 * i, c = j * 64 + lane;
		const int ci = c / P::PITCH_F4, f = c % P::PITCH_F4;
		const bool exists = j < P::ROW_LOADS && f < P::F4_ROW && ci < P::CIB && ci0 + ci < g.Cin;
		r_exists[i] = __ballot(exists);
		r_left[i] = __ballot(exists && f == 0);
		r_right[i] = __ballot(exists && f == P::F4_ROW - 1);
		r_voff[i] = exists ? (uint32_t)((ci * plane + 4 * f) * 4) : 0;  // from (row, column w0 - 4) of channel ci0
	}

	// ---- the load cursor: the chunk whose loads go out next, as (image, strip, row)
	int ld_n = begin / (tiles_w * g.H), ld_strip = (begin / g.H) % tiles_w, ld_ho = begin % g.H;
	auto advance = [&]() {
		if (++ld_ho == g.H) {
			ld_ho = 0;
			if (++ld_strip == tiles_w) {
				ld_strip = 0;
				ld_n++;
			}
		}
	};
	// one piece of the dy tile of the chunk under the cursor
	auto load_dy = [&](int stage, int k) {
		const float* dyb = dy + (((int64_t)ld_n * g.Cout + co0 + 16 * k) * g.H + ld_ho) * g.W + ld_strip * P::TW;
		async_load16_masked(dy_mask[k], smem_addr + stage * P::DY_BYTES + (4 * wave + k) * 1024, dyb, dy_voff);
	};
	// piece i of input row y (of the cursor's image and strip; -1 and H are the padding rows) into ring slot seq % 8
	auto load_row = [&](int y, int seq, int i) {
		const int w0 = ld_strip * P::TW;
		const float* xrow = x + (((int64_t)ld_n * g.Cin + ci0) * g.H + y) * g.W + w0 - 4;  // may lie before x: such lanes are masked
		const bool no_row = y < 0 || y >= g.H;
		const uint64_t outside = no_row ? r_exists[i] : ((w0 == 0 ? r_left[i] : 0) | (w0 + P::TW >= g.W ? r_right[i] : 0));
		const uint32_t slot = smem_addr + P::RING0 + (seq & (P::RING - 1)) * P::ROW_BYTES + (wave + 4 * i) * 1024;
		async_load16_masked(r_exists[i] & ~outside, slot, xrow, r_voff[i]);
		lds_zero16_masked(outside, slot + lane16, zero4);
	};
	constexpr int PIECES = P::DPW + P::RPW;

	// ---- the first chunk: its dy tile and all three rows
	int top_cur = 0, newest = 2;  // ring sequence numbers: of the current chunk's first row, of the last row fetched
	if (begin < end) {
#pragma unroll
		for (int k = 0; k < P::DPW; k++) load_dy(0, k);
#pragma unroll
		for (int r = 0; r < 3; r++)
#pragma unroll
			for (int i = 0; i < P::RPW; i++) load_row(ld_ho - 1 + r, r, i);
		advance();
	}

	v16f acc[P::TAPS];
#pragma unroll
	for (int t = 0; t < P::TAPS; t++)
#pragma unroll
		for (int r = 0; r < 16; r++) acc[t][r] = 0.0f;

	// operand addresses: a per-lane base plus immediates (the patch rows: plus the ring slot of each tap row)
	const int off_a = ((phalf * 8 + mt * 2 + (lrow >> 4)) * 1024) + (lrow & 15) * 16 + half * 4;
	const int off_b = P::RING0 + (lrow * P::CS + phalf * (P::TW / 2) + half + 3) * 4;

	wait_vmcnt_lgkm0<0>();
	__syncthreads();

	// MORE: a chunk follows (under the cursor), whose loads go out behind the first MFMAs
	auto run_chunk = [&](int cur, auto more_tag) {
		constexpr bool MORE = decltype(more_tag)::value;
		int top_next = top_cur + 1;
		if (MORE) {
			if (ld_ho == 0) {
				// first row of a strip: nothing of it is in the ring yet.  Two rows now, the third with the others below.
				top_next = newest + 1;
#pragma unroll
				for (int r = 0; r < 2; r++)
#pragma unroll
					for (int i = 0; i < P::RPW; i++) load_row(r - 1, top_next + r, i);
				newest += 2;
			}
			newest++;
		}
		const uint8_t* sa = smem + cur * P::DY_BYTES + off_a;
		const uint8_t* sb[3];
#pragma unroll
		for (int r = 0; r < 3; r++) sb[r] = smem + off_b + ((top_cur + r) & (P::RING - 1)) * P::ROW_BYTES;
		float fa[2], fb[2][P::TAPS];
		auto read_a = [&](int s) { fa[s & 1] = *reinterpret_cast<const float*>(sa + (s / 8) * 4096 + ((s / 2) % 4) * 256 + (s % 2) * 8); };
		auto read_b = [&](int s, int t) { fb[s & 1][t] = *reinterpret_cast<const float*>(sb[t / 3] + ((t % 3) + 2 * s) * 4); };
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
				if (MORE && k < P::DPW) load_dy(cur ^ 1, k);
				if (MORE && k >= P::DPW && k < PIECES) load_row(ld_ho + 1, newest, k - P::DPW);
				__builtin_amdgcn_sched_barrier(0);
			}
		}
		if (MORE) advance();
		top_cur = top_next;
		wait_vmcnt_lgkm0<0>();  // own loads of the next chunk have landed, own reads of this one are done
		__syncthreads();
	};
	int cur = 0;
	for (int chunk = begin; chunk + 1 < end; chunk++) {
		run_chunk(cur, std::true_type{});
		cur ^= 1;
	}
	if (begin < end) run_chunk(cur, std::false_type{});

	// pixel half 1 hands its sums to pixel half 0 of the same row tile
	float* lds = reinterpret_cast<float*>(smem);
	if (phalf == 1) {
#pragma unroll
		for (int t = 0; t < P::TAPS; t++)
#pragma unroll
			for (int r = 0; r < 16; r++) lds[((mt * P::TAPS + t) * 16 + r) * 64 + lane] = acc[t][r];
	}
	__syncthreads();
	if (phalf != 0) return;
#pragma unroll
	for (int t = 0; t < P::TAPS; t++)
#pragma unroll
		for (int r = 0; r < 16; r++) acc[t][r] += lds[((mt * P::TAPS + t) * 16 + r) * 64 + lane];

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
