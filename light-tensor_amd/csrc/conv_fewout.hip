// Conv2d forward, 3x3, stride 1, column padding 1, with at most four output channels — and through it the data
// gradient of a first layer (few input channels), which is such a convolution of dy with the flipped,
// channel-transposed weights.
//
// With so few output channels an MFMA tile would be almost empty (the 32-channel tile of the patch kernels spends
// 31/32 of its work on channels that do not exist when there is one); the work is a stream over x instead: every
// input value is read once from HBM and used for 9 * Cout multiply-adds.  A workgroup computes 8 rows x 128 columns
// of one image; a thread owns four consecutive pixels of one row and all output channels.  Input channels come in
// chunks of four: the patch [4 channels][10 rows][136 columns] (column q = input column w0 - 4 + q) is filled by
// direct global->LDS loads exactly as it lies in memory, two stages (on a 32-channel 128 x 128 data gradient at batch
// 32 a third stage is slower, 17.1 against 15.9 us).  Whether a float4 of the patch lies inside the image does not
// depend on the chunk: lanes whose float4 does not exist never load, and their slots keep the zeros written once.
// Per channel and patch row a thread needs six columns (4 t + 3 .. 4 t + 8): its own four in one 16-byte read, the two
// neighbours from the lanes beside it (a lane shift in the vector ALU), and multiplies them with the 3 * Cout
// weights of that row, which are wave-uniform and come through scalar loads.  DGRAD reads the weights of the transposed problem in place (w[ci][co][2 - i][2 - j]), so
// no flipped copy is made.
//
// Needs Cin % 4 == 0, W % 4 == 0 and 16-byte aligned x and y.
#include "conv_common.h"
#include "lds_async.h"

namespace lten_hip {

namespace {

struct FewOut {
	static constexpr int CB = 4, TH = 8, TW = 128, PR = TH + 2, PWS = 136, F4R = 34;
	static constexpr int PATCH_F4 = CB * PR * F4R;              // 1360
	static constexpr int LPW = (PATCH_F4 + 255) / 256;          // loads per wavefront and chunk: 6
	static constexpr int STAGE = LPW * 4 * 1024;                // bytes
	static constexpr int S = 2;                                 // stages: one chunk in flight while one is used
};

}  // namespace

template <int COUT, bool DGRAD>
__global__ __launch_bounds__(256) void conv2d_fewout_forward_kernel(ConvGeo g, const float* __restrict__ x, const float* __restrict__ w,
                                                                    const float* __restrict__ bias, float* __restrict__ y)
{
	typedef FewOut P;
	__shared__ __attribute__((aligned(1024))) uint8_t smem[P::S * P::STAGE];

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int trow = tid >> 5, tq = tid & 31;  // this thread's row of the tile and its group of four pixels
	const int tiles_w = (g.Wo + P::TW - 1) / P::TW;
	// Consecutive workgroup ids go round the eight XCDs: each XCD gets a contiguous run of (image, tile) items, so that
	// the tiles above and below a tile (two of its ten patch rows each) run on the same L2, close in time.  The grid is
	// 8 * per workgroups; the ones past the last item leave.
	const int tiles = tiles_w * ((g.Ho + P::TH - 1) / P::TH), total = tiles * g.N;
	const int per = (total + 7) / 8;
	const int item = ((int)blockIdx.x & 7) * per + ((int)blockIdx.x >> 3);
	if (item >= total) return;
	const int bx = item % tiles, n = item / tiles;
	const int w0 = (bx % tiles_w) * P::TW, h0 = (bx / tiles_w) * P::TH;
	const float* xn = x + (int64_t)n * g.Cin * g.H * g.W;

	// ---- what this lane fetches for each of its wavefront's loads (load q = wave + 4 i); always the same lanes
	uint32_t voff[P::LPW];
	uint64_t mask[P::LPW];
	const uint32_t smem_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
#pragma unroll
	for (int i = 0; i < P::LPW; i++) {
		const int idx = (wave + 4 * i) * 64 + lane;
		const int f = idx % P::F4R, r = (idx / P::F4R) % P::PR, c = idx / (P::F4R * P::PR);
		const int gy = h0 - g.ph + r, gx = w0 - 4 + 4 * f;
		const bool valid = idx < P::PATCH_F4 && gy >= 0 && gy < g.H && gx >= 0 && gx < g.W;
		voff[i] = valid ? (uint32_t)((((int64_t)c * g.H + gy) * g.W + gx) * 4) : 0;
		mask[i] = __ballot(valid);
	}
	// loads of this wavefront that fetch anything at all (a load whose lanes are all switched off may or may not
	// count as in flight; waiting for this many per chunk is right either way)
	int nload = 0;
#pragma unroll
	for (int i = 0; i < P::LPW; i++) nload += mask[i] != 0 ? 1 : 0;
	// waits until at most the loads of `chunks` chunks are in flight (loads return in order)
	auto wait_all_but = [&](int chunks) {
		switch (chunks * nload) {
		case 0: wait_vmcnt<0>(); break;
		case 1: wait_vmcnt<1>(); break;
		case 2: wait_vmcnt<2>(); break;
		case 3: wait_vmcnt<3>(); break;
		case 4: wait_vmcnt<4>(); break;
		case 5: wait_vmcnt<5>(); break;
		case 6: wait_vmcnt<6>(); break;
		case 8: wait_vmcnt<8>(); break;
		case 10: wait_vmcnt<10>(); break;
		default: wait_vmcnt<12>(); break;
		}
	};
	static_assert(P::LPW == 6 && P::S <= 3, "the switch above lists the products of 0..2 chunks and 0..6 loads");
	const int64_t x_step = (int64_t)P::CB * g.H * g.W;
	auto issue = [&](int stage, int kt) {
#pragma unroll
		for (int i = 0; i < P::LPW; i++) async_load16_masked(mask[i], smem_addr + stage * P::STAGE + (wave + 4 * i) * 1024, xn + kt * x_step, voff[i]);
	};

	// ---- zeros once in the slots no load ever writes (that is the padding): each lane clears its own, in every stage;
	// the slots that are loaded are never stored to, so the first loads need not wait for this
#pragma unroll
	for (int i = 0; i < P::LPW; i++) {
		const bool mine = !((mask[i] >> lane) & 1);
		if (mine)
#pragma unroll
			for (int st = 0; st < P::S; st++)
				*reinterpret_cast<float4*>(smem + st * P::STAGE + (wave + 4 * i) * 1024 + lane * 16) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
	}
	const int KT = g.Cin / P::CB;
#pragma unroll
	for (int st = 0; st < P::S; st++)
		if (st < KT) issue(st, st);

	float acc[COUT][4];
#pragma unroll
	for (int co = 0; co < COUT; co++)
#pragma unroll
		for (int j = 0; j < 4; j++) acc[co][j] = 0.0f;

	// columns 4 tq + 3 .. 4 tq + 8 of patch row trow + i hold input columns (w0 + 4 tq - 1) .. + 5
	const int off = (trow * P::PWS + 4 * tq + 3) * 4;
	int stage = 0;
	for (int kt = 0; kt < KT; kt++) {
		// this chunk's weights first (wave-uniform, scalar loads), so that they arrive while the patch is awaited
		float wt[P::CB][COUT][9];
#pragma unroll
		for (int c = 0; c < P::CB; c++)
#pragma unroll
			for (int co = 0; co < COUT; co++) {
				const int ci = kt * P::CB + c;
				const float* wr = DGRAD ? w + ((int64_t)ci * g.Cout + co) * 9 : w + ((int64_t)co * g.Cin + ci) * 9;
#pragma unroll
				for (int t = 0; t < 9; t++) wt[c][co][t] = DGRAD ? wr[8 - t] : wr[t];  // tap t = 3 i + j of the convolution computed here
			}
		wait_all_but(min(P::S - 1, KT - 1 - kt));  // chunk kt has landed; the chunks after it may still be on their way
		__syncthreads();
		const uint8_t* sbase = smem + stage * P::STAGE + off;
#pragma unroll
		for (int c = 0; c < P::CB; c++) {
#pragma unroll
			for (int i = 0; i < 3; i++) {
				const float* sp = reinterpret_cast<const float*>(sbase + ((c * P::PR + i) * P::PWS) * 4);
				// the four own columns in one read
				const float4 mid = *reinterpret_cast<const float4*>(sp + 1);
				// the neighbours' columns by a lane shift in the vector ALU (DPP wave_shr:1 / wave_shl:1: lane i takes lane
				// i - 1 / i + 1), and at the ends of the tile row from the patch: every lane reads its row's two edge values
				// (one address per row: a broadcast, no bank conflict) and keeps them only there — a branch around an LDS
				// read in the middle of the multiply-adds cost a fifth of the kernel's time
				float left = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(mid.w), 0x138, 0xf, 0xf, false));
				float right = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(mid.x), 0x130, 0xf, 0xf, false));
				const float* rowp = sp - 4 * tq;
				left = tq == 0 ? rowp[0] : left;
				right = tq == 31 ? rowp[4 * 31 + 5] : right;
				const float v[6] = { left, mid.x, mid.y, mid.z, mid.w, right };
#pragma unroll
				for (int co = 0; co < COUT; co++) {
#pragma unroll
					for (int j = 0; j < 3; j++) {
						const float wv = wt[c][co][3 * i + j];
#pragma unroll
						for (int p = 0; p < 4; p++) acc[co][p] = fmaf(v[p + j], wv, acc[co][p]);
					}
				}
			}
		}
		__syncthreads();  // everybody is done with this stage
		if (kt + P::S < KT) issue(stage, kt + P::S);
		stage = stage + 1 == P::S ? 0 : stage + 1;
	}

	const int ho = h0 + trow, wo = w0 + 4 * tq;
	if (ho >= g.Ho || wo >= g.Wo) return;
	const int64_t plane = (int64_t)g.Ho * g.Wo;
	float* yp = y + ((int64_t)n * g.Cout * g.Ho + ho) * g.Wo + wo;
#pragma unroll
	for (int co = 0; co < COUT; co++) {
		const float b = bias ? bias[co] : 0.0f;
		*reinterpret_cast<float4*>(yp + co * plane) = make_float4(acc[co][0] + b, acc[co][1] + b, acc[co][2] + b, acc[co][3] + b);
	}
}

bool conv_fewout_takes(const ConvGeo& g, const float* x, const float* y)
{
	return g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.kh == 3 && g.kw == 3 && g.pw == 1 && g.ph <= 2 && g.Cout >= 1 && g.Cout <= 4 &&
	       g.Cin % 4 == 0 && g.Cin >= 4 && g.W % 4 == 0 && aligned16(x) && aligned16(y) && (uint64_t)g.H * g.W < (1u << 26) && g.N < 65536 &&
	       ceil_div((uint64_t)g.Wo, 128) * ceil_div((uint64_t)g.Ho, 8) * g.N < (1u << 28);
}

// dgrad: w is the weight array of the convolution whose data gradient this is ([g.Cin][g.Cout][3][3] in terms of g)
template <bool DGRAD>
static int launch_fewout(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y)
{
	const uint64_t total = ceil_div((uint64_t)g.Wo, 128) * ceil_div((uint64_t)g.Ho, 8) * g.N;
	const dim3 grid((unsigned)(8 * ceil_div(total, 8))), block(256);
	switch (g.Cout) {
	case 1: conv2d_fewout_forward_kernel<1, DGRAD><<<grid, block, 0, stream()>>>(g, x, w, bias, y); break;
	case 2: conv2d_fewout_forward_kernel<2, DGRAD><<<grid, block, 0, stream()>>>(g, x, w, bias, y); break;
	case 3: conv2d_fewout_forward_kernel<3, DGRAD><<<grid, block, 0, stream()>>>(g, x, w, bias, y); break;
	default: conv2d_fewout_forward_kernel<4, DGRAD><<<grid, block, 0, stream()>>>(g, x, w, bias, y); break;
	}
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

int conv_fewout_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y, bool dgrad)
{
	set_kernel_name(dgrad ? "conv2d_fewout_dgrad_3x3_8x128" : "conv2d_fewout_forward_3x3_8x128");
	return dgrad ? launch_fewout<true>(g, x, w, bias, y) : launch_fewout<false>(g, x, w, bias, y);
}

}  // namespace lten_hip
