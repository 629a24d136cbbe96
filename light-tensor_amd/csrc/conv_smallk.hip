// Conv2d forward and weight gradient for stride 1, dilation 1 and a short reduction: Cin*kh*kw <= 32.
//
// This is the first layer of a network (l-ten/conv2d.cpp:164-171 with one or three input channels): almost no
// arithmetic, and y (forward) or dy (weight gradient) is the only large array.  Both kernels therefore touch
// y / dy exactly once with full rows per wavefront, keep the few input rows they need in LDS, and use one
// 32x32x2 fp32 MFMA tile whose reduction (forward) or column (weight gradient) dimension holds all taps.
//
// Work unit: a chunk = TW = 128 consecutive pixels of one output row of one image; the four wavefronts of a
// workgroup take 32 pixels each.  A workgroup walks a contiguous range of chunks with two LDS patch buffers:
// the rows of chunk c + 1 are fetched while chunk c is computed and stored to the other buffer after it, one barrier
// per chunk.  LDS patch row r = ci*kh + i holds input row ho + i - ph of channel ci, index q = input column
// w0 - 4 + q.
#include "conv_common.h"
#include "gemm_f32_core.h"

#include <algorithm>

namespace lten_hip {

namespace {

constexpr int SK_TW = 128;       // pixels per chunk
constexpr int SK_MAXK = 32;      // taps: one MFMA tile dimension
constexpr int SK_MAXKW = 9;      // widest kernel row the patch row has room for
constexpr int SK_PWS = 4 + SK_TW + SK_MAXKW - 1;  // 140 floats = 35 float4; 140 % 32 = 12 keeps 3x3 taps on 9 banks
constexpr int SK_F4_ROW = SK_PWS / 4;
constexpr int SK_PATCH = SK_MAXK * SK_PWS + 4;    // + a slot that stays zero (what padded taps read)
constexpr int SK_P_PER_T = (SK_MAXK * SK_F4_ROW + 255) / 256;
static_assert(SK_PWS % 4 == 0, "patch rows are whole float4s");

struct Chunk {
	int n, ho, w0;
};

__device__ __forceinline__ Chunk chunk_at(const ConvGeo& g, int chunk, int tiles_w)
{
	Chunk c;
	c.w0 = (chunk % tiles_w) * SK_TW;
	c.ho = (chunk / tiles_w) % g.Ho;
	c.n = chunk / (tiles_w * g.Ho);
	return c;
}

// This thread's share of the patch rows of a chunk: fetched to registers, stored to an LDS buffer later.
struct PatchRegs {
	float4 v[SK_P_PER_T];
};

template <bool VEC>
__device__ __forceinline__ void fetch_patch(const ConvGeo& g, const float* __restrict__ x, const Chunk& c, int tid, PatchRegs& p)
{
	const int rows = g.Cin * g.kh;
#pragma unroll
	for (int q = 0; q < SK_P_PER_T; q++) {
		const int idx = tid + q * 256;
		const int f = idx % SK_F4_ROW, r = idx / SK_F4_ROW;
		const int ci = r / g.kh, gy = c.ho + (r - ci * g.kh) - g.ph;
		p.v[q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
		if (r < rows && gy >= 0 && gy < g.H)
			p.v[q] = load_row4<VEC>(x + (((int64_t)c.n * g.Cin + ci) * g.H + gy) * g.W, c.w0 - 4 + 4 * f, g.W);
	}
}

__device__ __forceinline__ void store_patch(const ConvGeo& g, float* buf, int tid, const PatchRegs& p)
{
	const int rows = g.Cin * g.kh;
#pragma unroll
	for (int q = 0; q < SK_P_PER_T; q++) {
		const int idx = tid + q * 256;
		if (idx / SK_F4_ROW < rows) *reinterpret_cast<float4*>(buf + idx * 4) = p.v[q];
	}
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
template <bool VEC>
__global__ __launch_bounds__(256) void conv2d_smallk_forward_kernel(ConvGeo g, const float* __restrict__ x, const float* __restrict__ w,
                                                                    const float* __restrict__ bias, float* __restrict__ y, int chunks_per_group)
{
	__shared__ __attribute__((aligned(16))) float s_patch[2][SK_PATCH];
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lrow = lane & 31, half = lane >> 5;
	const int K = g.Cin * g.kh * g.kw, steps = (K + 1) / 2;
	const int co0 = blockIdx.y * 32;
	const int tiles_w = (g.Wo + SK_TW - 1) / SK_TW, total = g.N * g.Ho * tiles_w;
	const int begin = blockIdx.x * chunks_per_group, end = min(total, begin + chunks_per_group);
	if (begin >= end) return;

	if (tid < 4) { s_patch[0][SK_MAXK * SK_PWS + tid] = 0.0f; s_patch[1][SK_MAXK * SK_PWS + tid] = 0.0f; }

	// operand A: w[co0 + lrow][2s + half]; operand B address: this lane's pixel plus the tap offset
	const int pix = wave * 32 + lrow + 4 - g.pw;
	float wa[SK_MAXK / 2];
	int off[SK_MAXK / 2];
#pragma unroll
	for (int s = 0; s < SK_MAXK / 2; s++) {
		const int k = 2 * s + half;
		const bool valid = k < K;
		wa[s] = (valid && co0 + lrow < g.Cout) ? w[(int64_t)(co0 + lrow) * K + k] : 0.0f;
		off[s] = valid ? pix + tap_offset(g, k) : SK_MAXK * SK_PWS;
	}
	float bv[16];
#pragma unroll
	for (int r = 0; r < 16; r++) {
		const int co = co0 + (r >> 2) * 8 + half * 4 + (r & 3);
		bv[r] = (bias && co < g.Cout) ? bias[co] : 0.0f;
	}

	PatchRegs pr;
	fetch_patch<VEC>(g, x, chunk_at(g, begin, tiles_w), tid, pr);
	store_patch(g, s_patch[0], tid, pr);
	__syncthreads();
	for (int chunk = begin; chunk < end; chunk++) {
		const int cur = (chunk - begin) & 1;
		const Chunk c = chunk_at(g, chunk, tiles_w);
		if (chunk + 1 < end) fetch_patch<VEC>(g, x, chunk_at(g, chunk + 1, tiles_w), tid, pr);

		v16f acc;
#pragma unroll
		for (int r = 0; r < 16; r++) acc[r] = bv[r];
		const float* pb = s_patch[cur];
#pragma unroll
		for (int s = 0; s < SK_MAXK / 2; s++) {
			if (s >= steps) break;
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wa[s], pb[off[s]], acc, 0, 0, 0);
		}

		const int wo = c.w0 + wave * 32 + lrow;
		if (wo < g.Wo) {
#pragma unroll
			for (int r = 0; r < 16; r++) {
				const int co = co0 + (r >> 2) * 8 + half * 4 + (r & 3);
				if (co < g.Cout) y[(((int64_t)c.n * g.Cout + co) * g.Ho + c.ho) * g.Wo + wo] = acc[r];
			}
		}
		if (chunk + 1 < end) store_patch(g, s_patch[cur ^ 1], tid, pr);
		__syncthreads();
	}
}

// Weight gradient: dw[co][k] = sum over pixels of dy[co][pixel] * patch_k[pixel].  MFMA rows = 32 output
// channels, columns = taps (lanes whose column is >= K compute values nobody stores), reduction = the
// wavefront's 32 pixels of every chunk.  dy goes from global memory straight into the A operand: lane
// (co, half) loads four consecutive pixels at 8u + 4*half, so the 32-byte pieces a wavefront touches add up
// to whole rows over four loads.  Step (u, e) multiplies pixels 8u + e (lanes 0-31) and 8u + 4 + e (lanes 32-63).
template <bool VEC>
__global__ __launch_bounds__(256) void conv2d_smallk_wgrad_kernel(ConvGeo g, const float* __restrict__ x, const float* __restrict__ dy,
                                                                  float* __restrict__ partial, int chunks_per_part)
{
	__shared__ __attribute__((aligned(16))) float s_patch[2][SK_PATCH];
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lrow = lane & 31, half = lane >> 5;
	const int K = g.Cin * g.kh * g.kw;
	const int co0 = blockIdx.y * 32, co = co0 + lrow;
	const int tiles_w = (g.Wo + SK_TW - 1) / SK_TW, total = g.N * g.Ho * tiles_w;
	const int begin = blockIdx.x * chunks_per_part, end = min(total, begin + chunks_per_part);

	if (tid < 4) { s_patch[0][SK_MAXK * SK_PWS + tid] = 0.0f; s_patch[1][SK_MAXK * SK_PWS + tid] = 0.0f; }

	const int boff = (lrow < K ? tap_offset(g, lrow) : 0) + wave * 32 + 4 * half + 4 - g.pw;
	auto load_dy = [&](const Chunk& c, float4 (&a)[4]) {
#pragma unroll
		for (int u = 0; u < 4; u++) {
			a[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			if (co < g.Cout)
				a[u] = load_row4<VEC>(dy + (((int64_t)c.n * g.Cout + co) * g.Ho + c.ho) * g.Wo, c.w0 + wave * 32 + 8 * u + 4 * half, g.Wo);
		}
	};

	v16f acc;
#pragma unroll
	for (int r = 0; r < 16; r++) acc[r] = 0.0f;

	float4 a_cur[4], a_next[4];
	PatchRegs pr;
	if (begin < end) {
		const Chunk c = chunk_at(g, begin, tiles_w);
		fetch_patch<VEC>(g, x, c, tid, pr);
		load_dy(c, a_cur);
		store_patch(g, s_patch[0], tid, pr);
	}
	__syncthreads();
	for (int chunk = begin; chunk < end; chunk++) {
		const int cur = (chunk - begin) & 1;
		if (chunk + 1 < end) {
			const Chunk c = chunk_at(g, chunk + 1, tiles_w);
			fetch_patch<VEC>(g, x, c, tid, pr);
			load_dy(c, a_next);
		}
		const float* pb = s_patch[cur] + boff;
#pragma unroll
		for (int u = 0; u < 4; u++) {
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[u].x, pb[8 * u + 0], acc, 0, 0, 0);
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[u].y, pb[8 * u + 1], acc, 0, 0, 0);
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[u].z, pb[8 * u + 2], acc, 0, 0, 0);
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[u].w, pb[8 * u + 3], acc, 0, 0, 0);
		}
		if (chunk + 1 < end) {
			store_patch(g, s_patch[cur ^ 1], tid, pr);
#pragma unroll
			for (int u = 0; u < 4; u++) a_cur[u] = a_next[u];
		}
		__syncthreads();
	}

	// add the four wavefronts' tiles in wavefront order, then lanes whose column is a tap store
	float* red = &s_patch[0][0];
	if (wave != 0) {
#pragma unroll
		for (int r = 0; r < 16; r++) red[((wave - 1) * 16 + r) * 64 + lane] = acc[r];
	}
	__syncthreads();
	if (wave != 0 || lrow >= K) return;
	float* out = partial + (int64_t)blockIdx.x * g.Cout * K;
#pragma unroll
	for (int r = 0; r < 16; r++) {
		float v = acc[r];
#pragma unroll
		for (int q = 0; q < 3; q++) v += red[(q * 16 + r) * 64 + lane];
		const int row = co0 + (r >> 2) * 8 + half * 4 + (r & 3);
		if (row < g.Cout) out[(int64_t)row * K + lrow] = v;
	}
}

bool conv_smallk_takes(const ConvGeo& g)
{
	return g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.Cin * g.kh * g.kw <= SK_MAXK && g.kw <= SK_MAXKW && g.pw <= 4 &&
	       ceil_div((uint64_t)g.Cout, 32) < 65536 && (uint64_t)g.N * g.Ho * ceil_div((uint64_t)g.Wo, SK_TW) < (1ull << 31);
}

static uint64_t smallk_chunks(const ConvGeo& g) { return (uint64_t)g.N * g.Ho * ceil_div((uint64_t)g.Wo, SK_TW); }

// Workgroups along x: about four per CU over all channel blocks, at least two chunks each (none empty).
static int smallk_groups(const ConvGeo& g)
{
	const uint64_t chunks = smallk_chunks(g), blocks = ceil_div((uint64_t)g.Cout, 32);
	uint64_t groups = std::max<uint64_t>(1, 1024 / blocks);
	groups = std::min<uint64_t>(groups, std::max<uint64_t>(1, chunks / 2));
	const uint64_t per = ceil_div(chunks, groups);
	return (int)ceil_div(chunks, per);
}

int conv_smallk_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y)
{
	const int groups = smallk_groups(g);
	const int per = (int)ceil_div(smallk_chunks(g), (uint64_t)groups);
	const dim3 grid((unsigned)groups, (unsigned)ceil_div((uint64_t)g.Cout, 32));
	set_kernel_name("conv2d_smallk_forward_32x128");
	if (g.W % 4 == 0 && aligned16(x)) conv2d_smallk_forward_kernel<true><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y, per);
	else conv2d_smallk_forward_kernel<false><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y, per);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int conv_smallk_wgrad_parts(const ConvGeo& g) { return smallk_groups(g); }

int conv_smallk_wgrad(const ConvGeo& g, const float* x, const float* dy, float* partial, int parts)
{
	const int per = (int)ceil_div(smallk_chunks(g), (uint64_t)parts);
	const dim3 grid((unsigned)parts, (unsigned)ceil_div((uint64_t)g.Cout, 32));
	set_kernel_name("conv2d_smallk_wgrad_32x128");
	if (g.W % 4 == 0 && aligned16(x) && g.Wo % 4 == 0 && aligned16(dy))
		conv2d_smallk_wgrad_kernel<true><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per);
	else
		conv2d_smallk_wgrad_kernel<false><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, per);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // namespace lten_hip
