// Conv2d forward and weight gradient for stride 1, dilation 1 and a short reduction: Cin*kh*kw <= 32.
//
// This is the first layer of a network (l-ten/conv2d.cpp:164-171 with one or three input channels): almost no
// arithmetic, and y (forward) or dy (weight gradient) is the only large array.  Both kernels therefore touch
// y / dy exactly once with full rows per wavefront, keep the few input rows they need in LDS, and use one
// 32x32x2 fp32 MFMA tile whose reduction (forward) or column (weight gradient) dimension holds all taps.
//
// Work unit: a chunk = TW = 128 consecutive pixels of one output row of one image; the four wavefronts of a
// workgroup take 32 pixels each and never wait for one another: every wavefront keeps its own two LDS patch
// buffers (its 32 pixels plus the halo), fetches the rows of chunk c + 1 into registers while chunk c is
// computed, and stores them to the other buffer afterwards.  LDS operations of one wavefront complete in
// order, so no barrier separates a wavefront's patch stores from its own later reads.  LDS patch row
// r = ci*kh + i holds input row ho + i - ph of channel ci, index q = input column w0 + 32*wave - 4 + q.
#include "conv_common.h"
#include "gemm_f32_core.h"

#include <algorithm>

namespace lten_hip {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int SK_TW = 128;       // pixels per chunk
constexpr int SK_MAXK = 32;      // taps: one MFMA tile dimension
constexpr int SK_MAXKW = 9;      // widest kernel row the patch row has room for
constexpr int SK_PWS = 4 + 32 + SK_MAXKW - 1;     // 44 floats = 11 float4 per wavefront; 44 % 32 = 12 keeps 3x3 taps on 9 banks
constexpr int SK_F4_ROW = SK_PWS / 4;
static_assert(SK_PWS % 4 == 0, "patch rows are whole float4s");

// Two sizes of each kernel: RC = patch rows (Cin*kh) an LDS buffer has room for.  The small one (up to 8 rows
// and 16 taps, e.g. one input channel with a kernel of up to 4x4) keeps 9 KB of LDS and half the
// weight registers, so that more wavefronts share a CU and hide each other's load waits.
template <int RC>
struct SkShape {
	static constexpr int ROWS = RC;
	static constexpr int STEPS = RC <= 8 ? 8 : SK_MAXK / 2;  // MFMA steps (two taps each) held in registers
	static constexpr int ZERO = RC * SK_PWS;                  // a slot that stays zero (what padded taps read)
	static constexpr int PATCH = RC * SK_PWS + 4;
	static constexpr int P_PER_T = (RC * SK_F4_ROW + 63) / 64;  // float4 per lane
};

// Coordinates of a chunk.  A workgroup computes them once with divisions and then steps from chunk to chunk.
struct Chunk {
	int n, ho, w0;
};

// How a chunk's 128 pixels lie in the image: 128 columns of one row (a wavefront takes 32 of them), or, for narrow
// images, 32 columns of four rows (a wavefront takes a row): a 24-column image fills three quarters of such a chunk
// instead of a fifth.
struct Tiling {
	int cw, ch;           // columns and rows of a chunk
	int tiles_w, rows_c;  // chunks per image row and chunk rows per image
	int wx, wy;           // this wavefront's first column and its row inside the chunk
};

__device__ __forceinline__ Tiling make_tiling(const ConvGeo& g, int vert, int wave)
{
	Tiling t;
	t.cw = vert ? 32 : SK_TW;
	t.ch = vert ? 4 : 1;
	t.tiles_w = (g.Wo + t.cw - 1) / t.cw;
	t.rows_c = (g.Ho + t.ch - 1) / t.ch;
	t.wx = vert ? 0 : wave * 32;
	t.wy = vert ? wave : 0;
	return t;
}

__device__ __forceinline__ Chunk chunk_at(const Tiling& t, int chunk)
{
	Chunk c;
	c.w0 = (chunk % t.tiles_w) * t.cw;
	c.ho = ((chunk / t.tiles_w) % t.rows_c) * t.ch;
	c.n = chunk / (t.tiles_w * t.rows_c);
	return c;
}

__device__ __forceinline__ Chunk next_chunk(const ConvGeo& g, const Tiling& t, Chunk c)
{
	c.w0 += t.cw;
	if (c.w0 >= g.Wo) {
		c.w0 = 0;
		c.ho += t.ch;
		if (c.ho >= g.Ho) { c.ho = 0; c.n++; }
	}
	return c;
}

// This lane's share of its wavefront's patch rows: float4 number idx = lane + 64*q of the patch is column
// group f = idx % 11 of patch row r = idx / 11.  What does not change from chunk to chunk is worked out once:
// the offset of the row inside its image, and the row / column shifts that decide whether the piece lies
// inside the image.  The values are fetched to registers and stored to LDS later.
template <int P_PER_T>
struct PatchLane {
	int rel[P_PER_T];  // (ci*H + i - ph)*W + gx: element offset from x[n][0][ho][w0]
	int gy[P_PER_T];   // i - ph; far below -H for rows the geometry does not have
	int gx[P_PER_T];   // 32*wave - 4 + 4*f
	float4 v[P_PER_T];
};

template <int P_PER_T>
__device__ __forceinline__ void init_patch_lane(const ConvGeo& g, const Tiling& t, int lane, PatchLane<P_PER_T>& p)
{
	const int rows = g.Cin * g.kh;
#pragma unroll
	for (int q = 0; q < P_PER_T; q++) {
		const int idx = lane + q * 64;
		const int f = idx % SK_F4_ROW, r = idx / SK_F4_ROW;
		const int ci = r / g.kh, i = r - ci * g.kh;
		p.gx[q] = t.wx - 4 + 4 * f;
		p.gy[q] = r < rows ? t.wy + i - g.ph : -(1 << 30);
		p.rel[q] = r < rows ? (ci * g.H + t.wy + i - g.ph) * g.W + p.gx[q] : 0;
	}
}

template <bool VEC, int P_PER_T>
__device__ __forceinline__ void fetch_patch(const ConvGeo& g, const float* __restrict__ x, const Chunk& c, PatchLane<P_PER_T>& p)
{
	const float* origin = x + ((int64_t)c.n * g.Cin * g.H + c.ho) * g.W + c.w0;  // same for the whole workgroup
#pragma unroll
	for (int q = 0; q < P_PER_T; q++) {
		p.v[q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
		if ((unsigned)(c.ho + p.gy[q]) < (unsigned)g.H) {
			if (VEC) {  // W % 4 == 0 and gx % 4 == 0: the four columns are inside or outside together
				if ((unsigned)(c.w0 + p.gx[q]) < (unsigned)g.W) p.v[q] = *reinterpret_cast<const float4*>(origin + p.rel[q]);
			} else {
				p.v[q] = load_row4<false>(origin + (p.rel[q] - p.gx[q]) - c.w0, c.w0 + p.gx[q], g.W);
			}
		}
	}
}

template <int P_PER_T>
__device__ __forceinline__ void store_patch(float* buf, int lane, const PatchLane<P_PER_T>& p)
{
#pragma unroll
	for (int q = 0; q < P_PER_T; q++)
		if (p.gy[q] > -(1 << 29)) *reinterpret_cast<float4*>(buf + (lane + q * 64) * 4) = p.v[q];
}

// LDS offset of tap k = (ci, i, j) relative to the pixel's own position in patch row 0.
__device__ __forceinline__ int tap_offset(const ConvGeo& g, int k)
{
	const int j = k % g.kw, r = k / g.kw;  // r = ci*kh + i
	return r * SK_PWS + j;
}

}  // namespace

// Forward: y[n][co][ho][wo] = bias[co] + sum_k w[co][k] * patch_k[wo].  MFMA rows = 32 output channels
// (blockIdx.y picks the block), columns = the wavefront's 32 pixels, reduction = taps, two per step: lanes 0-31
// take tap 2s, lanes 32-63 tap 2s + 1.  The weights stay in registers for the whole kernel.
template <bool VEC, int RC>
__global__ __launch_bounds__(256) void conv2d_smallk_forward_kernel(ConvGeo g, const float* __restrict__ x, const float* __restrict__ w,
                                                                    const float* __restrict__ bias, float* __restrict__ y, int chunks_per_group, int vert)
{
	using S = SkShape<RC>;
	__shared__ __attribute__((aligned(16))) float s_mem[4 * 2 * S::PATCH];
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lrow = lane & 31, half = lane >> 5;
	const int K = g.Cin * g.kh * g.kw, steps = (K + 1) / 2;
	const int co0 = blockIdx.y * 32;
	const Tiling tl = make_tiling(g, vert, wave);
	const int total = g.N * tl.rows_c * tl.tiles_w;
	const int begin = blockIdx.x * chunks_per_group, end = min(total, begin + chunks_per_group);
	if (begin >= end) return;

	float* const mine = s_mem + wave * 2 * S::PATCH;  // this wavefront's two buffers
	if (lane < 4) { mine[S::ZERO + lane] = 0.0f; mine[S::PATCH + S::ZERO + lane] = 0.0f; }

	// operand A: w[co0 + lrow][2s + half]; operand B address: this lane's pixel plus the tap offset
	const int pix = lrow + 4 - g.pw;
	float wa[S::STEPS];
	int off[S::STEPS];
#pragma unroll
	for (int s = 0; s < S::STEPS; s++) {
		const int k = 2 * s + half;
		const bool valid = k < K;
		wa[s] = (valid && co0 + lrow < g.Cout) ? w[(int64_t)(co0 + lrow) * K + k] : 0.0f;
		off[s] = valid ? pix + tap_offset(g, k) : S::ZERO;
	}
	float bv[16];
#pragma unroll
	for (int r = 0; r < 16; r++) {
		const int co = co0 + (r >> 2) * 8 + half * 4 + (r & 3);
		bv[r] = (bias && co < g.Cout) ? bias[co] : 0.0f;
	}

	// stores: a row of y per register; the address is a part all lanes share plus this lane's offset
	const int64_t plane = (int64_t)g.Ho * g.Wo;
	const unsigned y_lane = (unsigned)(half * 4 * plane) + tl.wy * g.Wo + tl.wx + lrow;
	const bool all_channels = co0 + 32 <= g.Cout;

	PatchLane<S::P_PER_T> pr;
	init_patch_lane(g, tl, lane, pr);
	Chunk c = chunk_at(tl, begin);
	fetch_patch<VEC>(g, x, c, pr);
	store_patch(mine, lane, pr);
	for (int chunk = begin; chunk < end; chunk++) {
		const int cur = (chunk - begin) & 1;
		const Chunk nc = next_chunk(g, tl, c);
		if (chunk + 1 < end) fetch_patch<VEC>(g, x, nc, pr);

		v16f acc;
#pragma unroll
		for (int r = 0; r < 16; r++) acc[r] = bv[r];
		const float* pb = mine + cur * S::PATCH;
#pragma unroll
		for (int s = 0; s < S::STEPS; s++) {
			if (s >= steps) break;
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wa[s], pb[off[s]], acc, 0, 0, 0);
		}

		float* yc = y + (((int64_t)c.n * g.Cout + co0) * g.Ho + c.ho) * g.Wo + c.w0;  // same for the whole workgroup
		if (c.w0 + tl.wx + lrow < g.Wo && c.ho + tl.wy < g.Ho) {
			if (all_channels) {
#pragma unroll
				for (int r = 0; r < 16; r++) (yc + ((r >> 2) * 8 + (r & 3)) * plane)[y_lane] = acc[r];
			} else {
#pragma unroll
				for (int r = 0; r < 16; r++)
					if (co0 + (r >> 2) * 8 + half * 4 + (r & 3) < g.Cout) (yc + ((r >> 2) * 8 + (r & 3)) * plane)[y_lane] = acc[r];
			}
		}
		if (chunk + 1 < end) store_patch(mine + (cur ^ 1) * S::PATCH, lane, pr);
		c = nc;
	}
}

// Weight gradient: dw[co][k] = sum over pixels of dy[co][pixel] * patch_k[pixel].  MFMA rows = 32 output
// channels, columns = taps (lanes whose column is >= K compute values nobody stores), reduction = the
// wavefront's 32 pixels of every chunk.  Step (u, e) multiplies pixels 8u + e (lanes 0-31) and 8u + 4 + e
// (lanes 32-63), so lane (co, half) needs the four consecutive pixels at 8u + 4*half of row co.  With VEC the
// wavefront's 32 x 32 piece of dy is fetched as four loads of 8 rows x 128 bytes (whole cache lines: a load in the
// operand's own layout would touch 32 lines for 32 bytes each, and the line lookups, not the bytes, then set the
// pace) and turned into that layout through a wavefront-private LDS slab.
// WPG = 4 or 8 wavefronts per workgroup: with 8, wavefronts 4-7 take every other chunk of the workgroup's range, so
// that twice as many loads are in flight per CU for the same number of partial sums.
template <bool VEC, int RC, int WPG>
__global__ __launch_bounds__(WPG * 64) void conv2d_smallk_wgrad_kernel(ConvGeo g, const float* __restrict__ x, const float* __restrict__ dy,
                                                                  float* __restrict__ partial, int chunks_per_part, int vert)
{
	using S = SkShape<RC>;
	constexpr int RED = (WPG - 1) * 16 * 64;  // the other wavefronts' accumulator tiles for the final sum
	constexpr int DLD = 36, DSLAB = 32 * DLD;  // dy slab of a wavefront: [32 channels][32 pixels], rows of 36 floats
	constexpr int USED = WPG * 2 * S::PATCH + WPG * DSLAB;
	constexpr int STRIDE = WPG / 4;            // chunks between two of a wavefront's
	// At most 16 taps (a first layer with one input channel): 16x16x4 MFMA tiles, columns = taps, two row tiles of 16
	// channels, four pixels per step (lane l: tap or channel l % 16, pixel l / 16 of the step).  Half the matrix-pipe
	// time of the 32x32x2 tile, whose columns 16-31 would be padding.
	constexpr bool M16 = VEC && RC <= 8;
	__shared__ __attribute__((aligned(16))) float s_mem[USED > RED ? USED : RED];
	const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6, lrow = lane & 31, half = lane >> 5;
	const int l16 = lane & 15, kq = lane >> 4;
	const int wave = wid & 3;  // which 32 pixels of a chunk
	const int K = g.Cin * g.kh * g.kw;
	const int co0 = blockIdx.y * 32, co = co0 + lrow;
	const Tiling tl = make_tiling(g, vert, wave);
	const int total = g.N * tl.rows_c * tl.tiles_w;
	const int begin = blockIdx.x * chunks_per_part + (wid >> 2), end = min(total, (int)blockIdx.x * chunks_per_part + chunks_per_part);

	float* const mine = s_mem + wid * 2 * S::PATCH;  // this wavefront's two buffers
	float* const dslab = s_mem + WPG * 2 * S::PATCH + wid * DSLAB;
	const int r8 = lane >> 3, c4 = (lane & 7) * 4;     // whole-line loads: lane -> (row within a group of 8, 4 pixels)

	const int boff = M16 ? (l16 < K ? tap_offset(g, l16) : 0) + 4 * kq + 4 - g.pw : (lrow < K ? tap_offset(g, lrow) : 0) + 4 * half + 4 - g.pw;
	// dy: the address is a part all lanes share plus this lane's offset; with VEC (Wo % 4 == 0) the four
	// pixels of a load are inside or outside the row together
	const int64_t plane = (int64_t)g.Ho * g.Wo;
	const unsigned dy_lane = (VEC ? (unsigned)(r8 * plane) + c4 : (unsigned)(lrow * plane) + 4 * half) + tl.wy * g.Wo + tl.wx;
	const bool co_ok = co < g.Cout;
	// VEC: a[i] = rows 8i + r8, pixels c4 .. c4+3 (to be staged); else a[u] = the operand itself
	auto load_dy = [&](const Chunk& c, float4 (&a)[4]) {
		const float* dc = dy + (((int64_t)c.n * g.Cout + co0) * g.Ho + c.ho) * g.Wo + c.w0;  // same for the whole workgroup
		if (VEC) {
			const bool col_ok = c.w0 + tl.wx + c4 < g.Wo && c.ho + tl.wy < g.Ho;
#pragma unroll
			for (int i = 0; i < 4; i++) {
				a[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
				if (col_ok && co0 + 8 * i + r8 < g.Cout) a[i] = *reinterpret_cast<const float4*>(dc + 8 * i * plane + dy_lane);
			}
			return;
		}
		const int col = c.w0 + tl.wx + 4 * half;
#pragma unroll
		for (int u = 0; u < 4; u++) {
			a[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			if (co_ok && c.ho + tl.wy < g.Ho) a[u] = load_row4<false>(dc + dy_lane - (tl.wx + 4 * half) - c.w0, col + 8 * u, g.Wo);
		}
	};
	// VEC: through the slab into the operand layout
	auto stage_dy = [&](const float4 (&v)[4]) {
#pragma unroll
		for (int i = 0; i < 4; i++) *reinterpret_cast<float4*>(dslab + (8 * i + r8) * DLD + c4) = v[i];
	};
	// M16: a[2 ct + h] = channel 16 ct + l16, pixels 16 h + 4 kq .. + 3
	auto operand_dy = [&](float4 (&a)[4]) {
#pragma unroll
		for (int u = 0; u < 4; u++)
			a[u] = M16 ? *reinterpret_cast<const float4*>(dslab + (16 * (u >> 1) + l16) * DLD + 16 * (u & 1) + 4 * kq)
			           : *reinterpret_cast<const float4*>(dslab + lrow * DLD + 8 * u + 4 * half);
	};

	v16f acc;
#pragma unroll
	for (int r = 0; r < 16; r++) acc[r] = 0.0f;
	v4f acc16[2] = { { 0.0f, 0.0f, 0.0f, 0.0f }, { 0.0f, 0.0f, 0.0f, 0.0f } };

	float4 a_cur[4], a_next[4];
	PatchLane<S::P_PER_T> pr;
	init_patch_lane(g, tl, lane, pr);
	Chunk c = chunk_at(tl, begin);
	if (begin < end) {
		fetch_patch<VEC>(g, x, c, pr);
		load_dy(c, a_cur);
		store_patch(mine, lane, pr);
		if (VEC) stage_dy(a_cur);
	}
	for (int chunk = begin; chunk < end; chunk += STRIDE) {
		const int cur = ((chunk - begin) / STRIDE) & 1;
#pragma unroll
		for (int q = 0; q < STRIDE; q++) c = next_chunk(g, tl, c);
		if (chunk + STRIDE < end) {
			fetch_patch<VEC>(g, x, c, pr);
			load_dy(c, a_next);
		}
		if (VEC) operand_dy(a_cur);  // the slab is free again once these reads are issued (one wavefront, in order)
		const float* pb = mine + cur * S::PATCH + boff;
		if constexpr (M16) {
#pragma unroll
			for (int h = 0; h < 2; h++) {
				const float b0 = pb[16 * h + 0], b1 = pb[16 * h + 1], b2 = pb[16 * h + 2], b3 = pb[16 * h + 3];
#pragma unroll
				for (int ct = 0; ct < 2; ct++) {
					acc16[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_cur[2 * ct + h].x, b0, acc16[ct], 0, 0, 0);
					acc16[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_cur[2 * ct + h].y, b1, acc16[ct], 0, 0, 0);
					acc16[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_cur[2 * ct + h].z, b2, acc16[ct], 0, 0, 0);
					acc16[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_cur[2 * ct + h].w, b3, acc16[ct], 0, 0, 0);
				}
			}
		} else
#pragma unroll
		for (int u = 0; u < 4; u++) {
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[u].x, pb[8 * u + 0], acc, 0, 0, 0);
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[u].y, pb[8 * u + 1], acc, 0, 0, 0);
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[u].z, pb[8 * u + 2], acc, 0, 0, 0);
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[u].w, pb[8 * u + 3], acc, 0, 0, 0);
		}
		if (chunk + STRIDE < end) {
			store_patch(mine + (cur ^ 1) * S::PATCH, lane, pr);
			if (VEC) stage_dy(a_next);
			else {
#pragma unroll
				for (int u = 0; u < 4; u++) a_cur[u] = a_next[u];
			}
		}
	}

	// add the wavefronts' tiles in wavefront order, then lanes whose column is a tap store
	float* red = s_mem;
	__syncthreads();  // every wavefront is done with its patch buffers
	float* out = partial + (int64_t)blockIdx.x * g.Cout * K;
	if constexpr (M16) {
		// register r of tile ct in lane (l16, kq): channel 16 ct + 4 kq + r, tap l16
		if (wid != 0) {
#pragma unroll
			for (int r = 0; r < 8; r++) red[((wid - 1) * 8 + r) * 64 + lane] = acc16[r >> 2][r & 3];
		}
		__syncthreads();
		if (wid != 0 || l16 >= K) return;
#pragma unroll
		for (int r = 0; r < 8; r++) {
			float v = acc16[r >> 2][r & 3];
#pragma unroll
			for (int q = 0; q < WPG - 1; q++) v += red[(q * 8 + r) * 64 + lane];
			const int row = co0 + 16 * (r >> 2) + 4 * kq + (r & 3);
			if (row < g.Cout) out[(int64_t)row * K + l16] = v;
		}
		return;
	}
	if (wid != 0) {
#pragma unroll
		for (int r = 0; r < 16; r++) red[((wid - 1) * 16 + r) * 64 + lane] = acc[r];
	}
	__syncthreads();
	if (wid != 0 || lrow >= K) return;
#pragma unroll
	for (int r = 0; r < 16; r++) {
		float v = acc[r];
#pragma unroll
		for (int q = 0; q < WPG - 1; q++) v += red[(q * 16 + r) * 64 + lane];
		const int row = co0 + (r >> 2) * 8 + half * 4 + (r & 3);
		if (row < g.Cout) out[(int64_t)row * K + lrow] = v;
	}
}

bool conv_smallk_takes(const ConvGeo& g)
{
	return g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.Cin * g.kh * g.kw <= SK_MAXK && g.kw <= SK_MAXKW && g.pw <= 4 &&
	       (uint64_t)g.Ho * g.Wo <= (1u << 24) && (uint64_t)g.Cin * g.H * g.W < (1u << 29) &&  // 32-bit lane offsets
	       ceil_div((uint64_t)g.Cout, 32) < 65536 && (uint64_t)g.N * g.Ho * ceil_div((uint64_t)g.Wo, SK_TW) < (1ull << 31);
}

// The small kernel size: patch rows fit 8 and the taps fit 8 MFMA steps.
static bool smallk_small(const ConvGeo& g) { return g.Cin * g.kh <= 8 && g.Cin * g.kh * g.kw <= 16; }

// Chunks of four rows x 32 columns instead of 128 columns of one row, when that wastes clearly fewer pixels (l-ten's
// MNIST layer, 24 output columns: three quarters of a chunk are pixels instead of a fifth).
static bool smallk_vertical(const ConvGeo& g)
{
	const double wide = (double)g.Wo / (128.0 * (double)ceil_div((uint64_t)g.Wo, 128));
	const double tall = (double)g.Wo / (32.0 * (double)ceil_div((uint64_t)g.Wo, 32)) * (double)g.Ho / (4.0 * (double)ceil_div((uint64_t)g.Ho, 4));
	return tall > 1.15 * wide;
}

static uint64_t smallk_chunks(const ConvGeo& g)
{
	if (smallk_vertical(g)) return (uint64_t)g.N * ceil_div((uint64_t)g.Ho, 4) * ceil_div((uint64_t)g.Wo, 32);
	return (uint64_t)g.N * g.Ho * ceil_div((uint64_t)g.Wo, SK_TW);
}

// Workgroups along x: about `target` over all channel blocks, at least two chunks each (none empty).
static int smallk_groups(const ConvGeo& g, int target)
{
	const uint64_t chunks = smallk_chunks(g), blocks = ceil_div((uint64_t)g.Cout, 32);
	uint64_t groups = std::max<uint64_t>(1, (uint64_t)target / blocks);
	groups = std::min<uint64_t>(groups, std::max<uint64_t>(1, chunks / 2));
	const uint64_t per = ceil_div(chunks, groups);
	return (int)ceil_div(chunks, per);
}

int conv_smallk_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y)
{
	const int groups = smallk_groups(g, 1024);  // four workgroups per CU
	const int per = (int)ceil_div(smallk_chunks(g), (uint64_t)groups);
	const dim3 grid((unsigned)groups, (unsigned)ceil_div((uint64_t)g.Cout, 32));
	const bool vec = g.W % 4 == 0 && aligned16(x);
	const int vert = smallk_vertical(g) ? 1 : 0;
	if (smallk_small(g)) {
		set_kernel_name(vert ? "conv2d_smallk_forward_32x4x32_r8" : "conv2d_smallk_forward_32x128_r8");
		if (vec) conv2d_smallk_forward_kernel<true, 8><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y, per, vert);
		else conv2d_smallk_forward_kernel<false, 8><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y, per, vert);
	} else {
		set_kernel_name(vert ? "conv2d_smallk_forward_32x4x32" : "conv2d_smallk_forward_32x128");
		if (vec) conv2d_smallk_forward_kernel<true, SK_MAXK><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y, per, vert);
		else conv2d_smallk_forward_kernel<false, SK_MAXK><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y, per, vert);
	}
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// Two workgroups per CU: every workgroup leaves a partial sum that has to be written and read again.
int conv_smallk_wgrad_parts(const ConvGeo& g) { return smallk_groups(g, 512); }

int conv_smallk_wgrad(const ConvGeo& g, const float* x, const float* dy, float* partial, int parts)
{
	const int per = (int)ceil_div(smallk_chunks(g), (uint64_t)parts);
	const dim3 grid((unsigned)parts, (unsigned)ceil_div((uint64_t)g.Cout, 32));
	const bool vec = g.W % 4 == 0 && aligned16(x) && g.Wo % 4 == 0 && aligned16(dy);
	const int vert = smallk_vertical(g) ? 1 : 0;
	if (smallk_small(g)) {
		set_kernel_name(vert ? "conv2d_smallk_wgrad_32x4x32_r8" : "conv2d_smallk_wgrad_32x128_r8");
		if (vec) conv2d_smallk_wgrad_kernel<true, 8, 8><<<grid, dim3(512), 0, stream()>>>(g, x, dy, partial, per, vert);
		else conv2d_smallk_wgrad_kernel<false, 8, 4><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per, vert);
	} else {
		set_kernel_name(vert ? "conv2d_smallk_wgrad_32x4x32" : "conv2d_smallk_wgrad_32x128");
		if (vec) conv2d_smallk_wgrad_kernel<true, SK_MAXK, 4><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per, vert);
		else conv2d_smallk_wgrad_kernel<false, SK_MAXK, 4><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per, vert);
	}
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // namespace lten_hip
